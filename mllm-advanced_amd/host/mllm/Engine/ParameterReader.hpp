// The ".mllm" parameter container: 268-byte head, N x 416-byte descriptors, raw data
// (reference: mllm/Engine/ParameterReader.hpp:27-57 structs, ParameterReader.cpp:41-104 loader,
// :114-181 writer; the Python writer pads each tensor to 64 bytes, tools/convertor.py:173,207-211,
// which the offsets in the descriptors already account for).
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "mllm/Core/Tensor.hpp"

namespace mllm {

constexpr size_t kParameterNameLen = 256;
constexpr size_t kTensorShapeMaxLen = 16;
constexpr uint64_t kParameterMagicNumber = 0x519ACE0519ACE000ULL;

struct __attribute__((packed)) ParameterDescriptor {
  uint32_t parameter_id;
  uint32_t parameter_type;   // DataTypes code
  uint64_t parameter_size;   // bytes
  uint64_t parameter_offset; // from the start of the file
  uint64_t shape_len;
  uint64_t shape[kTensorShapeMaxLen];
  char name[kParameterNameLen];
};

struct __attribute__((packed)) ParameterPackHead {
  uint64_t magic_number;
  char model_name[kParameterNameLen];
  uint32_t parameter_cnt;
};

static_assert(sizeof(ParameterPackHead) == 268, "head is 268 bytes on disk");
static_assert(sizeof(ParameterDescriptor) == 416, "descriptor is 416 bytes on disk");

class ParameterLoader {
 public:
  ParameterLoader() = default;
  explicit ParameterLoader(const std::string& file_name);  // mmaps; tensors alias the mapping

  // Exits with kIOError if the name is missing, as the reference's table lookup would.
  std::shared_ptr<TensorViewImpl> operator[](const std::string& name);
  [[nodiscard]] bool has(const std::string& name) const { return params_.count(name) != 0; }
  std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>>& params() { return params_; }
  [[nodiscard]] const std::string& modelName() const { return model_name_; }

  // In-memory registration (what the quantizer does when it replaces a tensor).
  void insert(const std::string& name, const Tensor& t);

 private:
  std::shared_ptr<void> mapping_;
  std::string model_name_;
  std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>> params_;
};

std::shared_ptr<ParameterLoader> load(const std::string& file_path);

// Writes host tensors in the unpadded C++ layout of the reference writer.
void write(const std::shared_ptr<ParameterLoader>& params, const std::string& file_path,
           const std::string& model_name = "mllm");

}  // namespace mllm
