// What a device backend is to the engine (reference: mllm/Engine/BackendBase.hpp:20-46): a device
// key, an allocator and a table of op factories.
#pragma once

#include <memory>
#include <unordered_map>

#include "mllm/Core/AOps/BaseOp.hpp"
#include "mllm/Engine/Allocator.hpp"

namespace mllm {

class BackendBase {
 public:
  explicit BackendBase(DeviceTypes device) : device_(device) {}
  virtual ~BackendBase() = default;

  template <typename... Factories>
  void regOpFactory() {
    (..., regOne<Factories>());
  }

  [[nodiscard]] std::shared_ptr<Allocator> getAllocator() const { return allocator_; }
  std::shared_ptr<BaseOp> createOp(OpType op_type, const BaseOpCargoBase& base_cargo);
  [[nodiscard]] DeviceTypes deviceType() const { return device_; }

 private:
  template <typename T>
  void regOne() {
    auto f = std::make_shared<T>();
    op_factory_table_[static_cast<int>(f->opType())] = f;
  }

 protected:
  DeviceTypes device_;
  std::unordered_map<int, std::shared_ptr<BaseOpFactory>> op_factory_table_;
  std::shared_ptr<Allocator> allocator_ = nullptr;
};

}  // namespace mllm
