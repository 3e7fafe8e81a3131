// A contiguous tensor over reference-counted storage: the slice of the engine's Tensor that an
// operator boundary needs (reference: mllm/Core/Tensor.hpp:52-140, mllm/Core/TensorImpl.hpp:43-142).
// Tensor::empty() only describes a tensor; alloc() asks the device's allocator for memory, as
// BaseOp::setup does for op outputs (mllm/Core/AOps/BaseOp.cpp:25-46).
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "mllm/Core/DataTypes.hpp"
#include "mllm/Core/DeviceTypes.hpp"
#include "mllm/Engine/Allocator.hpp"

namespace mllm {

enum TensorMemTypes : int {  // NOLINT
  kNormal = 0,  // owned: freed through the allocator when the last reference goes
  kParams = 1,  // aliases a mapped parameter file or caller memory: never freed here
};

class TensorStorage : public Storage {
 public:
  ~TensorStorage() override;
  TensorMemTypes mem_type_ = kNormal;
  std::shared_ptr<void> keep_alive_;  // e.g. the mapped file a kParams tensor aliases
};

class TensorViewImpl {
 public:
  using shape_t = std::vector<int32_t>;
  shape_t shape_;
  DataTypes dtype_ = kFp32;
  std::string name_;
  std::shared_ptr<TensorStorage> storage_;
};

class Tensor {
 public:
  using shape_t = TensorViewImpl::shape_t;

  Tensor() = default;
  explicit Tensor(const std::shared_ptr<TensorViewImpl>& impl) : impl_(impl) {}

  [[nodiscard]] bool isNil() const { return impl_ == nullptr; }
  static Tensor nil() { return {}; }

  // Describes a tensor; no memory yet.
  static Tensor empty(const shape_t& shape, DataTypes dtype = kFp32, DeviceTypes device = kCPU);
  // Wraps memory owned by someone else (a mapped file, a caller's buffer).
  static Tensor wrap(void* ptr, const shape_t& shape, DataTypes dtype, DeviceTypes device,
                     std::shared_ptr<void> keep_alive = nullptr);

  Tensor& alloc();

  [[nodiscard]] const shape_t& shape() const { return impl_->shape_; }
  [[nodiscard]] DataTypes dtype() const { return impl_->dtype_; }
  [[nodiscard]] DeviceTypes device() const { return impl_->storage_->device_; }
  [[nodiscard]] size_t numel() const;
  [[nodiscard]] size_t bytes() const { return numel() * dataTypeSize(dtype()); }
  [[nodiscard]] const std::string& name() const { return impl_->name_; }
  void setName(const std::string& n) { impl_->name_ = n; }
  [[nodiscard]] const std::shared_ptr<TensorViewImpl>& impl() const { return impl_; }

  template <typename T>
  [[nodiscard]] T* ptr() const {
    return static_cast<T*>(impl_->storage_->ptr_);
  }

 private:
  std::shared_ptr<TensorViewImpl> impl_;
};

}  // namespace mllm
