// The MI355X backend: registers under kHIP, owns one HIP stream (default priority) and an
// allocator, and provides the op factories of the W4A32 decoder path. Shape of a GPU backend in the
// reference: mllm/Backends/CUDA/CUDABackend.cpp:18-24 (allocator + factory registration + D2H);
// the operator set follows mllm/Backends/Arm/ArmBackend.cpp:42-52.
//
// This directory uses only names that exist in the reference's headers plus DeviceTypes::kHIP.
#pragma once

#include <memory>
#include <vector>

#include "mllm/Core/Tensor.hpp"
#include "mllm/Engine/BackendBase.hpp"
#include "mllm/Utils/Common.hpp"

namespace mllm::hip {

// Exit code for a failed HIP runtime or kernel-library call: the reference's one code for a GPU runtime
// failure (mllm/Utils/Common.hpp:29), so that no enumerator has to be added there.
inline constexpr ExitCode kHipRuntimeError = ExitCode::kCudaError;

// Bytes a (dense) tensor's elements occupy. Tensor::bytes() is not const in the reference
// (mllm/Core/Tensor.hpp:439) and operators receive their inputs as const references.
inline size_t tensorBytes(const Tensor& t) { return t.numel() * dataTypeSize(t.dtype()); }

// hipMalloc-backed allocator, 256-byte alignment (the kernels want 16-byte aligned blobs and
// 256-byte aligned workspaces). Reference counterpart: mllm/Backends/CUDA/CUDAAllocator.cpp.
// ctrlByMllmMemManager() is true: the engine's memory manager asks it for blocks and hands them out
// again itself, so a tensor's birth and death do not reach hipMalloc / hipFree.
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

// malloc-backed host allocator for a process that registers no CPU backend of the engine's own.
class HostAllocator final : public Allocator {
 public:
  bool ctrlByMllmMemManager() override { return false; }
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
  ~HipBackend();  // BackendBase has no virtual destructor: hold a HipBackend through make_shared's pointer

  [[nodiscard]] void* stream() const { return stream_; }  // hipStream_t
  void synchronize() const;

  // Device memory that an op may use while its kernels run (partial sums of a product whose k range is
  // dealt to several workgroups): one buffer for the backend, grown on demand, contents undefined. All ops
  // run in order on the backend's one stream, so the next borrower cannot overlap the previous one.
  Tensor& scratch(size_t bytes);

  // RoPE sin / cos tables [max_pos][dims / 2] on the device, built once per (theta, max_pos, dims) and
  // shared by every RoPE op (the reference shares its tables through global tensors, RoPEOp.cpp:20-50).
  void ropeTables(float theta, int max_pos, int dims, Tensor* sin, Tensor* cos);

 private:
  struct RopeTables {
    float theta;
    int max_pos, dims;
    Tensor sin, cos;
  };
  void* stream_ = nullptr;
  Tensor scratch_;
  std::vector<RopeTables> rope_tables_;
};

std::shared_ptr<HipBackend> createHipBackend();
std::shared_ptr<HostBackend> createHostBackend();

// The registered HIP backend (exits if there is none).
HipBackend& currentHipBackend();

// Host <-> device copies on the backend's stream. toHost synchronises before returning
// (the reference's host consumers read the tensor right after a D2H op).
Tensor toDevice(const Tensor& host);
Tensor toHost(const Tensor& device);

// A host parameter as an f32 device tensor of the same shape: Fp32 is copied, Fp16 (how the reference's W4A32
// quantizer configuration stores the RMSNorm weights, scripts/QuantCfg/ds_qwen2/1.5B-W4A32-KAI.json:33-42) is
// widened on the device, exactly. Any other dtype exits.
Tensor toDeviceF32(const Tensor& host);

}  // namespace mllm::hip
