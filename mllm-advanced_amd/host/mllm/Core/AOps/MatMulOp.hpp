// Outside the reference tree this name forwards to the engine slice the HIP backend is built against.
#pragma once
#include "mllm/EngineSlice.hpp"
