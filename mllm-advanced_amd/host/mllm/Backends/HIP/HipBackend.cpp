#include "mllm/Backends/HIP/HipBackend.hpp"

#include <hip/hip_runtime_api.h>

#include <cstdlib>
#include <cstring>

#include "mllm/Backends/HIP/Ops/DecoderOps.hpp"
#include "mllm/Backends/HIP/Ops/LinearOp.hpp"
#include "mllm/Engine/Context.hpp"
#include "mllm/Utils/Log.hpp"
#include "w4a32_decoder.h"

#define MLLM_CHECK_HIP(expr)                                                                         \
  do {                                                                                               \
    hipError_t e_ = (expr);                                                                          \
    if (e_ != hipSuccess) {                                                                          \
      MLLM_ERROR_EXIT(::mllm::hip::kHipRuntimeError, "{} failed: {}", #expr, hipGetErrorString(e_)); \
    }                                                                                                \
  } while (0)

namespace mllm::hip {

namespace {
size_t roundUp(size_t v, size_t a) { return (v + a - 1) / a * a; }
}  // namespace

bool HipAllocator::alloc(const std::shared_ptr<Storage>& storage) {
  void* p = nullptr;
  if (!generalAlloc(&p, storage->size_, alignSize()) || !p) return false;
  storage->ptr_ = p;
  return true;
}

void HipAllocator::free(Storage* storage) { generalFree(storage->ptr_); }

bool HipAllocator::generalAlloc(void** ptr, size_t cap, size_t align) {
  const size_t bytes = roundUp(cap ? cap : 1, align);
  MLLM_CHECK_HIP(hipMalloc(ptr, bytes));  // hipMalloc returns memory aligned to 256 bytes or more
  return *ptr != nullptr;
}

void HipAllocator::generalFree(void* ptr) {
  if (!ptr) return;
  MLLM_CHECK_HIP(hipDeviceSynchronize());  // the stream may still be using it
  MLLM_CHECK_HIP(hipFree(ptr));
}

size_t HipAllocator::allocSize(Storage* storage) { return roundUp(storage->size_, alignSize()); }

bool HostAllocator::alloc(const std::shared_ptr<Storage>& storage) {
  void* p = nullptr;
  if (!generalAlloc(&p, storage->size_, alignSize())) return false;
  storage->ptr_ = p;
  return true;
}

void HostAllocator::free(Storage* storage) { generalFree(storage->ptr_); }

bool HostAllocator::generalAlloc(void** ptr, size_t cap, size_t align) {
  *ptr = std::aligned_alloc(align, roundUp(cap ? cap : 1, align));
  return *ptr != nullptr;
}

void HostAllocator::generalFree(void* ptr) { std::free(ptr); }

size_t HostAllocator::allocSize(Storage* storage) { return roundUp(storage->size_, alignSize()); }

HostBackend::HostBackend() : BackendBase(kCPU) { allocator_ = std::make_shared<HostAllocator>(); }

HipBackend::HipBackend() : BackendBase(kHIP) {
  int count = 0;
  MLLM_CHECK_HIP(hipGetDeviceCount(&count));
  if (count < 1) { MLLM_ERROR_EXIT(kHipRuntimeError, "no HIP device is visible"); }
  MLLM_CHECK_HIP(hipSetDevice(0));
  hipDeviceProp_t prop{};
  MLLM_CHECK_HIP(hipGetDeviceProperties(&prop, 0));
  MLLM_INFO("Found device: {} ({}, {} CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
  hipStream_t s = nullptr;
  MLLM_CHECK_HIP(hipStreamCreate(&s));  // default priority
  stream_ = s;
  allocator_ = std::make_shared<HipAllocator>();
  regOpFactory<HipLinearOpFactory, HipD2HOpFactory, HipViewOpFactory, HipRMSNormOpFactory, HipRoPEOpFactory,
               HipKVCacheOpFactory, HipFlashAttn2OpFactory, HipMatMulOpFactory, HipSiLUOpFactory, HipAddOpFactory,
               HipMulOpFactory, HipLLMEmbeddingTokenOpFactory>();
}

HipBackend::~HipBackend() {
  if (stream_) {
    (void)hipStreamSynchronize(static_cast<hipStream_t>(stream_));
    (void)hipStreamDestroy(static_cast<hipStream_t>(stream_));
  }
}

Tensor& HipBackend::scratch(size_t bytes) {
  if (scratch_.isNil() || tensorBytes(scratch_) < bytes) {
    scratch_ = Tensor::empty({static_cast<int32_t>(bytes)}, kInt8, kHIP).alloc();
  }
  return scratch_;
}

void HipBackend::ropeTables(float theta, int max_pos, int dims, Tensor* sin, Tensor* cos) {
  for (auto& t : rope_tables_) {
    if (t.theta == theta && t.max_pos == max_pos && t.dims == dims) {
      *sin = t.sin;
      *cos = t.cos;
      return;
    }
  }
  RopeTables t{theta, max_pos, dims, Tensor::empty({max_pos, dims / 2}, kFp32, kHIP).alloc(),
               Tensor::empty({max_pos, dims / 2}, kFp32, kHIP).alloc()};
  const int rc = w4a32_op_rope_table(t.sin.ptr<float>(), t.cos.ptr<float>(), max_pos, dims, theta, stream_);
  if (rc != W4A32_OK) { MLLM_ERROR_EXIT(kHipRuntimeError, "w4a32_op_rope_table failed: {}", w4a32_error_string(rc)); }
  rope_tables_.push_back(t);
  *sin = t.sin;
  *cos = t.cos;
}

void HipBackend::synchronize() const {
  MLLM_CHECK_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream_)));
}

std::shared_ptr<HipBackend> createHipBackend() { return std::make_shared<HipBackend>(); }
std::shared_ptr<HostBackend> createHostBackend() { return std::make_shared<HostBackend>(); }

HipBackend& currentHipBackend() {
  // BackendBase is not polymorphic: the device key is what identifies the backend registered under it
  std::shared_ptr<BackendBase> b = MllmEngineCtx::instance().getBackend(kHIP);
  if (!b || b->deviceType() != kHIP) { MLLM_ERROR_EXIT(kError, "no HIP backend is registered"); }
  return *static_cast<HipBackend*>(b.get());
}

Tensor toDevice(const Tensor& host) {
  MLLM_RT_ASSERT(host.device() == kCPU);
  Tensor d = Tensor::empty(host.shape(), host.dtype(), kHIP).alloc();
  d.setName(host.name());
  auto s = static_cast<hipStream_t>(currentHipBackend().stream());
  MLLM_CHECK_HIP(hipMemcpyAsync(d.ptr<char>(), host.ptr<char>(), tensorBytes(host), hipMemcpyHostToDevice, s));
  MLLM_CHECK_HIP(hipStreamSynchronize(s));  // the source may be pageable or go away
  return d;
}

Tensor toDeviceF32(const Tensor& host) {
  if (host.dtype() == kFp32) return toDevice(host);
  if (host.dtype() != kFp16) {
    MLLM_ERROR_EXIT(kError, "{}: expected an Fp32 or Fp16 parameter, got {}", host.name(), dataTypes2Str(host.dtype()));
  }
  Tensor half = toDevice(host);
  Tensor d = Tensor::empty(host.shape(), kFp32, kHIP).alloc();
  d.setName(host.name());
  auto& hb = currentHipBackend();
  const int rc = w4a32_op_f16_to_f32(half.ptr<void>(), d.ptr<float>(), host.numel(), hb.stream());
  if (rc != W4A32_OK) { MLLM_ERROR_EXIT(kHipRuntimeError, "w4a32_op_f16_to_f32 failed: {}", w4a32_error_string(rc)); }
  hb.synchronize();  // `half` is released on return
  return d;
}

Tensor toHost(const Tensor& device) {
  MLLM_RT_ASSERT(device.device() == kHIP);
  Tensor h = Tensor::empty(device.shape(), device.dtype(), kCPU).alloc();
  h.setName(device.name());
  auto s = static_cast<hipStream_t>(currentHipBackend().stream());
  MLLM_CHECK_HIP(hipMemcpyAsync(h.ptr<char>(), device.ptr<char>(), tensorBytes(device), hipMemcpyDeviceToHost, s));
  MLLM_CHECK_HIP(hipStreamSynchronize(s));
  return h;
}

}  // namespace mllm::hip
