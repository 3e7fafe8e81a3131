// Allocator interface a backend hands to the engine (reference: mllm/Engine/Allocator.hpp:18-32,
// same nine virtuals with the same meaning).
#pragma once

#include <cstddef>
#include <memory>

#include "mllm/Core/DeviceTypes.hpp"

namespace mllm {

// reference: mllm/Core/Storage.hpp:20-37
class Storage : public std::enable_shared_from_this<Storage> {
 public:
  virtual ~Storage() = default;
  void* ptr_ = nullptr;
  size_t size_ = 0;
  DeviceTypes device_ = kCPU;
};

class Allocator {
 public:
  virtual ~Allocator() = default;
  virtual bool ctrlByMllmMemManager() = 0;
  virtual bool alloc(const std::shared_ptr<Storage>& storage) = 0;
  virtual void free(const std::shared_ptr<Storage>& storage) = 0;
  virtual void free(Storage* storage) = 0;
  virtual bool generalAlloc(void** ptr, size_t cap, size_t align) = 0;
  virtual void generalFree(void* ptr) = 0;
  virtual size_t allocSize(Storage* storage) = 0;
  virtual size_t allocSize(const std::shared_ptr<Storage>& storage) = 0;
  [[nodiscard]] virtual size_t alignSize() const = 0;
};

}  // namespace mllm
