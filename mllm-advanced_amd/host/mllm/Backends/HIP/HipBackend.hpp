// The MI355X backend: registers under kHIP, owns one HIP stream (default priority) and an
// allocator, and provides the Linear and D2H op factories. Shape of a GPU backend in the
// reference: mllm/Backends/CUDA/CUDABackend.cpp:18-24 (allocator + factory registration + D2H).
#pragma once

#include <memory>

#include "mllm/Core/Tensor.hpp"
#include "mllm/Engine/BackendBase.hpp"

namespace mllm::hip {

// hipMalloc-backed allocator, 256-byte alignment (the kernels want 16-byte aligned blobs and
// 256-byte aligned workspaces). Reference counterpart: mllm/Backends/CUDA/CUDAAllocator.cpp.
class HipAllocator final : public Allocator {
 public:
  bool ctrlByMllmMemManager() override { return true; }
  bool alloc(const std::shared_ptr<Storage>& storage) override;
  void free(const std::shared_ptr<Storage>& storage) override { free(storage.get()); }
  void free(Storage* storage) override;
  bool generalAlloc(void** ptr, size_t cap, size_t align) override;
  void generalFree(void* ptr) override;
  size_t allocSize(Storage* storage) override;
  size_t allocSize(const std::shared_ptr<Storage>& storage) override { return allocSize(storage.get()); }
  [[nodiscard]] size_t alignSize() const override { return 256; }
};

// malloc-backed host allocator so host tensors can be created through the same Tensor API.
class HostAllocator final : public Allocator {
 public:
  bool ctrlByMllmMemManager() override { return true; }
  bool alloc(const std::shared_ptr<Storage>& storage) override;
  void free(const std::shared_ptr<Storage>& storage) override { free(storage.get()); }
  void free(Storage* storage) override;
  bool generalAlloc(void** ptr, size_t cap, size_t align) override;
  void generalFree(void* ptr) override;
  size_t allocSize(Storage* storage) override;
  size_t allocSize(const std::shared_ptr<Storage>& storage) override { return allocSize(storage.get()); }
  [[nodiscard]] size_t alignSize() const override { return 64; }
};

class HostBackend final : public BackendBase {
 public:
  HostBackend();
};

class HipBackend final : public BackendBase {
 public:
  HipBackend();
  ~HipBackend() override;

  [[nodiscard]] void* stream() const { return stream_; }  // hipStream_t
  void synchronize() const;

  // Device memory that an op may use while its kernels run (partial sums of a product whose k range is
  // dealt to several workgroups): one buffer for the backend, grown on demand, contents undefined. All ops
  // run in order on the backend's one stream, so the next borrower cannot overlap the previous one.
  Tensor& scratch(size_t bytes);

 private:
  void* stream_ = nullptr;
  Tensor scratch_;
};

std::shared_ptr<HipBackend> createHipBackend();
std::shared_ptr<HostBackend> createHostBackend();

// The registered HIP backend (exits if there is none).
HipBackend& currentHipBackend();

// Host <-> device copies on the backend's stream. toHost synchronises before returning
// (the reference's host consumers read the tensor right after a D2H op).
Tensor toDevice(const Tensor& host);
Tensor toHost(const Tensor& device);

}  // namespace mllm::hip
