// The element types this path touches, with the numeric codes the .mllm container stores
// (reference: mllm/Core/DataTypes.hpp:19-65 - Int8 = 2, Int32 = 4, Int64 = 5, Fp16 = 8, Fp32 = 9, BF16 = 24).
#pragma once

#include <cstddef>
#include <cstdint>

namespace mllm {

enum DataTypes : uint32_t {  // NOLINT
  kInt8 = 2,
  kInt32 = 4,
  kInt64 = 5,
  kFp16 = 8,
  kFp32 = 9,
  kBF16 = 24,
};

inline size_t dataTypeSize(DataTypes t) {
  switch (t) {
    case kInt8: return 1;
    case kFp16:
    case kBF16: return 2;
    case kInt32:
    case kFp32: return 4;
    case kInt64: return 8;
  }
  return 0;
}

inline const char* dataTypes2Str(DataTypes t) {
  switch (t) {
    case kInt8: return "Int8";
    case kInt32: return "Int32";
    case kInt64: return "Int64";
    case kFp16: return "Fp16";
    case kFp32: return "Fp32";
    case kBF16: return "BF16";
  }
  return "Unknown";
}

}  // namespace mllm
