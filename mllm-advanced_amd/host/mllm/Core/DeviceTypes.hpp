// Device enum of the engine, with the one value this backend adds.
// Reference: mllm/Core/DeviceTypes.hpp:18-27 has kCPU, kCUDA, kOpenCL, kQNN; a backend is looked
// up by this key (mllm/Engine/Context.cpp:56-59), so a new device needs a new enumerator: kHIP.
#pragma once

#include <string>

namespace mllm {

enum DeviceTypes {  // NOLINT
  kDeviceTypes_Start = 0,
  kCPU,
  kCUDA,
  kOpenCL,
  kQNN,
  kHIP,  // added: AMD GPU through HIP (MI355X / gfx950)
  kDeviceTypes_End,
};

inline const char* deviceTypes2Str(DeviceTypes t) {
  static const char* const names[] = {"DeviceTypes_Start", "CPU", "CUDA", "OpenCL", "QNN", "HIP",
                                      "DeviceTypes_End"};
  return (t >= kDeviceTypes_Start && t <= kDeviceTypes_End) ? names[t] : "Unknown";
}

inline DeviceTypes str2DeviceType(const std::string& s) {
  for (int t = kCPU; t < kDeviceTypes_End; ++t) {
    if (s == deviceTypes2Str(static_cast<DeviceTypes>(t))) return static_cast<DeviceTypes>(t);
  }
  return kDeviceTypes_End;
}

}  // namespace mllm
