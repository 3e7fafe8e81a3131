#include "mllm/Backends/HIP/Ops/LinearOp.hpp"

#include <hip/hip_runtime_api.h>

#include <cstring>

#include "mllm/Backends/HIP/HipBackend.hpp"
#include "mllm/Engine/Context.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "mllm/Utils/Log.hpp"
#include "w4a32_hip.h"

namespace mllm::hip {

namespace {

void check(int rc, const char* what) {
  if (rc != W4A32_OK) { MLLM_ERROR_EXIT(kHipRuntimeError, "{} failed: {}", what, w4a32_error_string(rc)); }
}

void checkHip(hipError_t e, const char* what) {
  if (e != hipSuccess) { MLLM_ERROR_EXIT(kHipRuntimeError, "{} failed: {}", what, hipGetErrorString(e)); }
}

// The six tile variants of KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk (values 3..8 of LinearOpImplType,
// mllm/Core/AOps/LinearOp.hpp:21-26): the one family this backend implements.
bool isW4A32ImplType(LinearOpImplType t) {
  const int v = static_cast<int>(t);
  return v >= 3 && v <= 8;
}

// Packing parameters of the reference's six W4A32 tiles (ukernel table kai_linear.cpp:123-218): nr
// from "qsi4c32p<nr>x..", kr / sr from the micro-kernel family (p4x8, p8x8: 16 / 2; p4x4: 8 / 2).
// [parity unpinned: KleidiAI, which defines them, is not part of the reference tree]
struct KaiTile {
  int nr, kr, sr;
};
KaiTile kaiTile(LinearOpImplType t) {
  switch (static_cast<int>(t)) {
    case 4:
    case 7: return {8, 16, 2};
    case 8: return {4, 8, 2};
    default: return {4, 16, 2};
  }
}

}  // namespace

HipLinearOp::HipLinearOp(const LinearOpCargo& cargo) : LinearOp(cargo) {}

size_t HipLinearOp::nativeBlobBytes(int N, int K) {
  return w4a32_native_u4_bytes(N, K) + w4a32_native_scale_bytes(N, K) + (size_t)N * sizeof(float);
}

void HipLinearOp::load(const std::shared_ptr<ParameterLoader>& ploader) {
  const int N = cargo_.out_channels, K = cargo_.in_channels;
  if (!isW4A32ImplType(cargo_.impl_type_)) {
    MLLM_ERROR_EXIT(kError, "{}: the HIP backend implements the W4A32 Linear family only "
                    "(KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk:*), impl type {} asked",
                    name(), static_cast<int>(cargo_.impl_type_));
    return;
  }
  const size_t packed_bytes = w4a32_packed_bytes(N, K);
  if (packed_bytes == 0) {
    MLLM_ERROR_EXIT(kError, "{}: in_channels {} must be a positive multiple of 32", name(), K);
    return;
  }
  LinearOp::load(ploader);  // weight_/bias_ now alias the (host) parameter file
  auto& hb = currentHipBackend();
  void* stream = hb.stream();
  Tensor packed = Tensor::empty({static_cast<int32_t>(packed_bytes)}, kInt8, kHIP).alloc();

  if ((weight_.dtype() == kFp32 || weight_.dtype() == kFp16) && weight_.shape().size() == 2 &&
      weight_.shape()[0] == N && weight_.shape()[1] == K) {
    // an unquantised weight (f32, or f16 widened exactly): quantised here, as the reference's offline pass would
    Tensor w_dev = toDeviceF32(weight_);
    Tensor b_dev;
    if (cargo_.bias) {
      if ((bias_.dtype() != kFp32 && bias_.dtype() != kFp16) || static_cast<int>(bias_.numel()) != N) {
        MLLM_ERROR_EXIT(kError, "{}.bias must be f32 or f16 [{}]", name(), N);
        return;
      }
      b_dev = toDeviceF32(bias_);
    }
    const size_t tmp_bytes = w4a32_native_u4_bytes(N, K) + w4a32_native_scale_bytes(N, K);
    Tensor tmp = Tensor::empty({static_cast<int32_t>(tmp_bytes)}, kInt8, kHIP).alloc();
    check(w4a32_quant_pack_rhs(w_dev.ptr<float>(), b_dev.isNil() ? nullptr : b_dev.ptr<float>(), N, K,
                               packed.ptr<void>(), tmp.ptr<void>(), W4A32_BF16_TRUNC, stream),
          "w4a32_quant_pack_rhs");
    hb.synchronize();  // tmp, w_dev, b_dev are released on return
  } else if (weight_.dtype() == kInt8 && weight_.numel() == nativeBlobBytes(N, K)) {
    Tensor blob = toDevice(weight_);
    const size_t u4_bytes = w4a32_native_u4_bytes(N, K), sc_bytes = w4a32_native_scale_bytes(N, K);
    const uint8_t* u4 = blob.ptr<uint8_t>();
    const auto* sc = reinterpret_cast<const uint16_t*>(u4 + u4_bytes);
    // The f32 bias follows the bf16 scales, so it is only 2-byte aligned when N * K/32 is odd (both in
    // the file and in its device copy): the kernel gets a copy of its own, aligned like any tensor.
    Tensor bias_host = Tensor::empty({N}, kFp32, kCPU).alloc();
    std::memcpy(bias_host.ptr<char>(), weight_.ptr<char>() + u4_bytes + sc_bytes, (size_t)N * sizeof(float));
    Tensor bias_dev = toDevice(bias_host);
    check(w4a32_repack_native(u4, sc, bias_dev.ptr<float>(), N, K, packed.ptr<void>(), stream),
          "w4a32_repack_native");
    hb.synchronize();
  } else if (const KaiTile kt = kaiTile(cargo_.impl_type_);
             weight_.dtype() == kInt8 && weight_.numel() == w4a32_kai_blob_bytes(N, K, kt.nr)) {
    // The blob the reference's Arm quantizer wrote for this tile (KaiQuantizationPass.cpp:172-184):
    // un-interleave it to the native arrays, then repack. Its bias sits inside the blob (the
    // file's <name>.bias is a 1-byte placeholder). Layout restated from KleidiAI: parity unpinned.
    Tensor blob = toDevice(weight_);
    const size_t u4_bytes = w4a32_native_u4_bytes(N, K), sc_bytes = w4a32_native_scale_bytes(N, K);
    Tensor tmp = Tensor::empty({static_cast<int32_t>(u4_bytes + sc_bytes + (size_t)N * sizeof(float))},
                               kInt8, kHIP).alloc();
    uint8_t* u4 = tmp.ptr<uint8_t>();
    auto* sc = reinterpret_cast<uint16_t*>(u4 + u4_bytes);
    auto* bias = reinterpret_cast<float*>(u4 + u4_bytes + sc_bytes);
    check(w4a32_unpack_kai(blob.ptr<void>(), N, K, kt.nr, kt.kr, kt.sr, u4, sc, bias, stream),
          "w4a32_unpack_kai");
    check(w4a32_repack_native(u4, sc, bias, N, K, packed.ptr<void>(), stream), "w4a32_repack_native");
    hb.synchronize();
  } else {
    MLLM_ERROR_EXIT(kError, "{}.weight: expected f32 / f16 [{},{}] or an int8 W4 blob of {} bytes, "
                    "got {} with {} elements", name(), N, K, nativeBlobBytes(N, K),
                    dataTypes2Str(weight_.dtype()), weight_.numel());
    return;
  }
  packed.setName(name() + ".weight");
  weight_ = packed;  // the op now holds the device blob; the host tensors are dropped
  bias_ = Tensor::nil();
}

void HipLinearOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& i = inputs[0];
  auto o_shape = i.shape();
  MLLM_RT_ASSERT_EQ(o_shape[o_shape.size() - 1], cargo_.in_channels);
  o_shape[o_shape.size() - 1] = cargo_.out_channels;
  // the W4A32 family always produces f32 (reference Arm/Ops/LinearOp.cpp:253-260)
  outputs.emplace_back(Tensor::empty(o_shape, kFp32, i.device()));
}

void HipLinearOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& x = inputs[0];
  auto& y = outputs[0];
  if (x.device() != kHIP || x.dtype() != kFp32) {
    MLLM_ERROR_EXIT(kError, "{}: input must be an f32 tensor on the HIP device", name());
    return;
  }
  if (weight_.isNil() || weight_.device() != kHIP) {
    MLLM_ERROR_EXIT(kError, "{}: forward before load", name());
    return;
  }
  const int K = cargo_.in_channels, N = cargo_.out_channels;
  // Every leading dimension is a row. (The reference reads M = shape[-2] and ignores the others,
  // Arm/Ops/LinearOp.cpp:68; the engine only ever runs batch 1, where the two agree.)
  const int M = static_cast<int>(x.numel() / static_cast<size_t>(K));
  // The workspace holds the quantised rows and, behind them, room for the partial sums of a product whose k
  // range the library deals to several workgroups (few output tiles and a long K: down_proj at prefill sizes).
  const size_t need = w4a32_workspace_bytes_n(M, K, N);
  if (workspace_.isNil() || tensorBytes(workspace_) < need) {
    workspace_ = Tensor::empty({static_cast<int32_t>(need)}, kInt8, kHIP).alloc();
  }
  auto& hb = currentHipBackend();
  check(w4a32_matmul_ws(y.ptr<float>(), x.ptr<float>(), weight_.ptr<void>(), workspace_.ptr<void>(),
                        tensorBytes(workspace_), M, K, N, hb.stream()),
        "w4a32_matmul_ws");
  // Stays asynchronous on the backend's stream: a host consumer goes through D2H, which waits.
}

HipD2HOp::HipD2HOp(const D2HOpCargo& cargo) : D2HOp(cargo) {}

void HipD2HOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  auto s = static_cast<hipStream_t>(currentHipBackend().stream());
  checkHip(hipMemcpyAsync(outputs[0].ptr<char>(), inputs[0].ptr<char>(), tensorBytes(inputs[0]),
                          hipMemcpyDeviceToHost, s), "hipMemcpyAsync(D2H)");
  checkHip(hipStreamSynchronize(s), "hipStreamSynchronize");
}

Tensor quantizeLinearForFile(const Tensor& weight_f32, const Tensor& bias_f32_or_nil) {
  MLLM_RT_ASSERT(weight_f32.dtype() == kFp32 && weight_f32.shape().size() == 2);
  const int N = weight_f32.shape()[0], K = weight_f32.shape()[1];
  const size_t u4_bytes = w4a32_native_u4_bytes(N, K), sc_bytes = w4a32_native_scale_bytes(N, K);
  if (u4_bytes == 0) {
    MLLM_ERROR_EXIT(kError, "quantize: in_channels {} must be a positive multiple of 32", K);
    return Tensor::nil();
  }
  auto& hb = currentHipBackend();
  Tensor w_dev = toDevice(weight_f32);
  Tensor planes = Tensor::empty({static_cast<int32_t>(u4_bytes + sc_bytes)}, kInt8, kHIP).alloc();
  check(w4a32_quant_rhs_native(w_dev.ptr<float>(), N, K, planes.ptr<uint8_t>(),
                               reinterpret_cast<uint16_t*>(planes.ptr<uint8_t>() + u4_bytes),
                               W4A32_BF16_TRUNC, hb.stream()),
        "w4a32_quant_rhs_native");
  Tensor planes_host = toHost(planes);
  Tensor blob = Tensor::empty({static_cast<int32_t>(HipLinearOp::nativeBlobBytes(N, K))}, kInt8, kCPU).alloc();
  std::memcpy(blob.ptr<uint8_t>(), planes_host.ptr<uint8_t>(), u4_bytes + sc_bytes);
  auto* bias_out = reinterpret_cast<float*>(blob.ptr<uint8_t>() + u4_bytes + sc_bytes);
  if (bias_f32_or_nil.isNil()) {
    std::memset(bias_out, 0, (size_t)N * sizeof(float));
  } else {
    MLLM_RT_ASSERT(bias_f32_or_nil.dtype() == kFp32 && static_cast<int>(bias_f32_or_nil.numel()) == N);
    std::memcpy(bias_out, bias_f32_or_nil.ptr<float>(), (size_t)N * sizeof(float));
  }
  return blob;
}

}  // namespace mllm::hip
