// The extern "C" surface declared in include/w4a32_hip.h: argument checks, geometry,
// dispatch to the launchers. Nothing here allocates, frees or synchronises.
#include "w4a32_hip.h"

#include "w4a32_internal.h"

namespace {

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline int shape_ok(int N, int K) {
  if (N <= 0 || K <= 0) return W4A32_EINVAL;
  if (K % w4::kBlockLen != 0) return W4A32_ESHAPE;
  return W4A32_OK;
}

inline int from_hip(hipError_t e) { return e == hipSuccess ? W4A32_OK : W4A32_ELAUNCH; }

constexpr int kMaxDevices = 64;

}  // namespace

// Activation workspace of w4a32_matmul_static_ws: one copy per GPU, part of the code object's
// zero-initialised data, held until the process ends. In host code this name only identifies the
// symbol; the memory's address on a device comes from hipGetSymbolAddress (static_ws_ptr below).
static __device__ __align__(256) unsigned char scratch[W4A32_STATIC_WS_BYTES];

namespace {

// Address of `scratch` on each device, looked up on the first call made with that device current.
std::atomic<void*> g_static_ws[kMaxDevices];

int static_ws_ptr(void** out, hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return W4A32_ELAUNCH;
  if (dev < 0 || dev >= kMaxDevices) return W4A32_ENOTSUP;
  void* p = g_static_ws[dev].load(std::memory_order_acquire);
  if (!p) {
    // The lookup is a runtime query, not stream work: it does not belong into a capture. A first call on a
    // capturing stream is refused before anything is launched, so the capture stays valid and empty-handed.
    if (stream) {
      hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
      if (hipStreamIsCapturing(stream, &st) != hipSuccess) return W4A32_ELAUNCH;
      if (st != hipStreamCaptureStatusNone) return W4A32_ENOTSUP;
    }
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return W4A32_ELAUNCH;
    g_static_ws[dev].store(p, std::memory_order_release);  // racing first calls store the same address
  }
  *out = p;
  return W4A32_OK;
}

}  // namespace

extern "C" {

const char* w4a32_error_string(int code) {
  switch (code) {
    case W4A32_OK: return "ok";
    case W4A32_EINVAL: return "invalid argument (null/misaligned pointer or non-positive size)";
    case W4A32_ESHAPE: return "unsupported shape (K must be a multiple of 32; M must fit the kernel)";
    case W4A32_ELAUNCH: return "HIP launch failed";
    case W4A32_ENOTSUP: return "not supported by this build";
    case W4A32_ETOOBIG: return "rows need more than the static workspace (W4A32_STATIC_WS_BYTES)";
    default: return "unknown error";
  }
}

int w4a32_abi_version(void) { return 1; }

size_t w4a32_packed_bytes(int N, int K) {
  if (shape_ok(N, K) != W4A32_OK) return 0;
  return w4::weight_geom(N, K).total_bytes;
}

size_t w4a32_workspace_bytes(int M, int K) {
  if (M <= 0 || shape_ok(1, K) != W4A32_OK) return 0;
  return w4::ws_geom(M, K).total_bytes;
}

size_t w4a32_native_u4_bytes(int N, int K) {
  if (shape_ok(N, K) != W4A32_OK) return 0;
  return (size_t)N * (K / 2);
}

size_t w4a32_native_scale_bytes(int N, int K) {
  if (shape_ok(N, K) != W4A32_OK) return 0;
  return (size_t)N * (K / w4::kBlockLen) * sizeof(uint16_t);
}

int w4a32_quant_rhs_native(const float* d_w, int N, int K, uint8_t* d_u4, uint16_t* d_scales,
                           int bf16_mode, void* stream) {
  if (int e = shape_ok(N, K)) return e;
  if (!d_w || !d_u4 || !d_scales) return W4A32_EINVAL;
  if (!aligned(d_w, 16) || !aligned(d_u4, 16) || !aligned(d_scales, 2)) return W4A32_EINVAL;
  if (bf16_mode != W4A32_BF16_TRUNC && bf16_mode != W4A32_BF16_RNE) return W4A32_EINVAL;
  return from_hip(w4::launch_quant_rhs(d_w, N, K, d_u4, d_scales, bf16_mode,
                                       static_cast<hipStream_t>(stream)));
}

int w4a32_repack_native(const uint8_t* d_u4, const uint16_t* d_scales, const float* d_bias, int N,
                        int K, void* d_packed, void* stream) {
  if (int e = shape_ok(N, K)) return e;
  if (!d_u4 || !d_scales || !d_packed) return W4A32_EINVAL;
  if (!aligned(d_u4, 16) || !aligned(d_scales, 2) || !aligned(d_packed, 16)) return W4A32_EINVAL;
  return from_hip(w4::launch_repack(d_u4, d_scales, d_bias, N, K, static_cast<uint8_t*>(d_packed),
                                    static_cast<hipStream_t>(stream)));
}

int w4a32_quant_pack_rhs(const float* d_w, const float* d_bias, int N, int K, void* d_packed,
                         void* d_tmp, int bf16_mode, void* stream) {
  if (int e = shape_ok(N, K)) return e;
  if (!d_tmp || !aligned(d_tmp, 16)) return W4A32_EINVAL;
  uint8_t* u4 = static_cast<uint8_t*>(d_tmp);
  uint16_t* sc = reinterpret_cast<uint16_t*>(u4 + w4a32_native_u4_bytes(N, K));
  if (int e = w4a32_quant_rhs_native(d_w, N, K, u4, sc, bf16_mode, stream)) return e;
  return w4a32_repack_native(u4, sc, d_bias, N, K, d_packed, stream);
}

int w4a32_unpack_native(const void* d_packed, int N, int K, uint8_t* d_u4, uint16_t* d_scales,
                        float* d_bias, void* stream) {
  if (int e = shape_ok(N, K)) return e;
  if (!d_packed || !d_u4 || !d_scales) return W4A32_EINVAL;
  if (!aligned(d_packed, 16) || !aligned(d_u4, 4) || !aligned(d_scales, 2)) return W4A32_EINVAL;
  return from_hip(w4::launch_unpack(static_cast<const uint8_t*>(d_packed), N, K, d_u4, d_scales,
                                    d_bias, static_cast<hipStream_t>(stream)));
}

size_t w4a32_kai_blob_bytes(int N, int K, int nr) {
  if (shape_ok(N, K) || (nr != 4 && nr != 8)) return 0;
  return (size_t)((N + nr - 1) / nr) * nr * ((size_t)(K / 32) * 18 + 8);
}

int w4a32_unpack_kai(const void* d_kai_blob, int N, int K, int nr, int kr, int sr, uint8_t* d_u4,
                     uint16_t* d_scales, float* d_bias, void* stream) {
  if (int e = shape_ok(N, K)) return e;
  if (!d_kai_blob || !d_u4 || !d_scales) return W4A32_EINVAL;
  if ((nr != 4 && nr != 8) || sr <= 0 || kr <= 0 || kr % sr != 0) return W4A32_EINVAL;
  const int seg = kr / sr;
  if (seg != 4 && seg != 8 && seg != 16) return W4A32_EINVAL;  // a segment divides half a block
  return from_hip(w4::launch_unpack_kai(static_cast<const uint8_t*>(d_kai_blob), N, K, nr, kr, sr, d_u4,
                                        d_scales, d_bias, static_cast<hipStream_t>(stream)));
}

int w4a32_dequant(const void* d_packed, int N, int K, float* d_out, void* stream) {
  if (int e = shape_ok(N, K)) return e;
  if (!d_packed || !d_out) return W4A32_EINVAL;
  if (!aligned(d_packed, 16) || !aligned(d_out, 16)) return W4A32_EINVAL;
  return from_hip(w4::launch_dequant(static_cast<const uint8_t*>(d_packed), N, K, d_out,
                                     static_cast<hipStream_t>(stream)));
}

int w4a32_quant_lhs(const float* d_x, int M, int K, int ldx, void* d_ws, void* stream) {
  if (M <= 0) return W4A32_EINVAL;
  if (int e = shape_ok(1, K)) return e;
  if (!d_x || !d_ws || ldx < K) return W4A32_EINVAL;
  if (!aligned(d_x, 16) || (ldx % 4) != 0 || !aligned(d_ws, 256)) return W4A32_EINVAL;
  return from_hip(w4::launch_quant_lhs(d_x, M, K, ldx, static_cast<uint8_t*>(d_ws),
                                       static_cast<hipStream_t>(stream)));
}

int w4a32_export_lhs(const void* d_ws, int M, int K, int8_t* d_aq, float* d_recip_scale,
                     int32_t* d_neg_zero_point, void* stream) {
  if (M <= 0) return W4A32_EINVAL;
  if (int e = shape_ok(1, K)) return e;
  if (!d_ws || !d_aq || !d_recip_scale || !d_neg_zero_point) return W4A32_EINVAL;
  const w4::WsGeom g = w4::ws_geom(M, K);
  const uint8_t* ws = static_cast<const uint8_t*>(d_ws);
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e = hipMemcpyAsync(d_aq, ws + g.aq_off, (size_t)M * K, hipMemcpyDeviceToDevice, s);
  if (e == hipSuccess)
    e = hipMemcpyAsync(d_recip_scale, ws + g.scale_off, (size_t)M * 4, hipMemcpyDeviceToDevice, s);
  if (e == hipSuccess)
    e = hipMemcpyAsync(d_neg_zero_point, ws + g.off_off, (size_t)M * 4, hipMemcpyDeviceToDevice, s);
  return from_hip(e);
}

int w4a32_matmul_quantized_ex(float* d_y, const void* d_ws, const void* d_packed, int M, int K,
                              int N, int kernel, void* stream) {
  if (M <= 0) return W4A32_EINVAL;
  if (int e = shape_ok(N, K)) return e;
  if (!d_y || !d_ws || !d_packed) return W4A32_EINVAL;
  if (!aligned(d_ws, 256) || !aligned(d_packed, 16) || !aligned(d_y, 4)) return W4A32_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint8_t* ws = static_cast<const uint8_t*>(d_ws);
  const uint8_t* pk = static_cast<const uint8_t*>(d_packed);
  switch (kernel) {
    case W4A32_KERNEL_AUTO:
      if (M <= w4::kGemvMaxM) return from_hip(w4::launch_gemv(d_y, ws, pk, M, K, N, s));
      return from_hip(w4::launch_gemm(d_y, ws, pk, M, K, N, w4::kKernelAuto, s));
    case W4A32_KERNEL_GEMV:
      if (M > w4::kGemvMaxM) return W4A32_ESHAPE;
      return from_hip(w4::launch_gemv(d_y, ws, pk, M, K, N, s));
    case W4A32_KERNEL_GEMM_I8:
      return from_hip(w4::launch_gemm(d_y, ws, pk, M, K, N, w4::kKernelGemmI8, s));
    case W4A32_KERNEL_GEMM_F16:
      if (M <= w4::kGemvMaxM) return W4A32_ESHAPE;  // the f16 activation copy exists only for M > 8
      return from_hip(w4::launch_gemm(d_y, ws, pk, M, K, N, w4::kKernelGemmF16, s));
    default:
      if (kernel >= W4A32_KERNEL_GEMM_F16_TILE0 &&
          kernel < W4A32_KERNEL_GEMM_F16_TILE0 + W4A32_GEMM_F16_TILES) {
        if (M <= w4::kGemvMaxM) return W4A32_ESHAPE;
        return from_hip(w4::launch_gemm(d_y, ws, pk, M, K, N, kernel, s));
      }
      return W4A32_EINVAL;
  }
}

size_t w4a32_splitk_scratch_bytes(int M, int K, int N) {
  if (M <= w4::kGemvMaxM || shape_ok(N, K)) return 0;
  const w4::SplitPlan p = w4::splitk_plan(M, K, N);
  return p.parts > 1 ? (size_t)p.parts * M * N * sizeof(float) : 0;
}

int w4a32_matmul_quantized_splitk(float* d_y, const void* d_ws, const void* d_packed, int M, int K,
                                  int N, void* d_scratch, size_t scratch_bytes, void* stream) {
  const size_t need = w4a32_splitk_scratch_bytes(M, K, N);
  if (need == 0 || !d_scratch || scratch_bytes < need) {
    return w4a32_matmul_quantized(d_y, d_ws, d_packed, M, K, N, stream);
  }
  if (!d_y || !d_ws || !d_packed) return W4A32_EINVAL;
  if (!aligned(d_ws, 256) || !aligned(d_packed, 16) || !aligned(d_y, 16) || !aligned(d_scratch, 16)) {
    return W4A32_EINVAL;
  }
  return from_hip(w4::launch_gemm_splitk(d_y, static_cast<const uint8_t*>(d_ws),
                                         static_cast<const uint8_t*>(d_packed), M, K, N,
                                         static_cast<float*>(d_scratch), static_cast<hipStream_t>(stream)));
}

int w4a32_matmul_quantized(float* d_y, const void* d_ws, const void* d_packed, int M, int K, int N,
                           void* stream) {
  return w4a32_matmul_quantized_ex(d_y, d_ws, d_packed, M, K, N, W4A32_KERNEL_AUTO, stream);
}

int w4a32_matmul(float* d_y, const float* d_x, const void* d_packed, void* d_ws, int M, int K,
                 int N, void* stream) {
  if (M > 0 && shape_ok(N, K) == W4A32_OK && w4::gemv_fused_applies(M, K, N)) {
    // decode sizes: one kernel quantises the rows and multiplies (the workspace stays unused)
    if (!d_y || !d_x || !d_packed || !d_ws) return W4A32_EINVAL;
    if (!aligned(d_x, 16) || !aligned(d_packed, 16) || !aligned(d_y, 4)) return W4A32_EINVAL;
    return from_hip(w4::launch_gemv_fused(d_y, d_x, K, static_cast<const uint8_t*>(d_packed), M, K,
                                          N, static_cast<hipStream_t>(stream)));
  }
  if (int e = w4a32_quant_lhs(d_x, M, K, K, d_ws, stream)) return e;
  return w4a32_matmul_quantized(d_y, d_ws, d_packed, M, K, N, stream);
}

size_t w4a32_workspace_bytes_n(int M, int K, int N) {
  const size_t ws = w4a32_workspace_bytes(M, K);
  if (ws == 0 || shape_ok(N, K)) return 0;
  return w4::round_up_sz(ws, 256) + w4a32_splitk_scratch_bytes(M, K, N);
}

int w4a32_matmul_ws(float* d_y, const float* d_x, const void* d_packed, void* d_ws, size_t ws_bytes, int M,
                    int K, int N, void* stream) {
  if (M <= 0) return W4A32_EINVAL;
  if (int e = shape_ok(N, K)) return e;
  const size_t ws = w4a32_workspace_bytes(M, K);
  if (!d_ws || ws_bytes < ws) return W4A32_EINVAL;
  const size_t parts = w4a32_splitk_scratch_bytes(M, K, N), parts_off = w4::round_up_sz(ws, 256);
  if (parts != 0 && ws_bytes >= parts_off + parts && aligned(d_y, 16)) {
    if (int e = w4a32_quant_lhs(d_x, M, K, K, d_ws, stream)) return e;
    return w4a32_matmul_quantized_splitk(d_y, d_ws, d_packed, M, K, N, static_cast<uint8_t*>(d_ws) + parts_off,
                                         parts, stream);
  }
  return w4a32_matmul(d_y, d_x, d_packed, d_ws, M, K, N, stream);
}

int w4a32_matmul_static_ws(float* d_y, const float* d_x, const void* d_packed, int M, int K, int N,
                           void* stream) {
  if (M <= 0) return W4A32_EINVAL;
  if (int e = shape_ok(N, K)) return e;
  if (w4::ws_geom(M, K).total_bytes > (size_t)W4A32_STATIC_WS_BYTES) return W4A32_ETOOBIG;
  void* ws = nullptr;
  if (int e = static_ws_ptr(&ws, static_cast<hipStream_t>(stream))) return e;
  return w4a32_matmul(d_y, d_x, d_packed, ws, M, K, N, stream);
}

int w4a32_matmul_grouped(float* const* d_y, const float* d_x, const void* const* d_packed,
                         const int* N, int count, void* d_ws, int M, int K, void* stream) {
  if (!d_y || !d_x || !d_packed || !N || !d_ws) return W4A32_EINVAL;
  if (count < 1 || count > W4A32_MAX_GROUP || M <= 0) return W4A32_EINVAL;
  for (int i = 0; i < count; ++i) {
    if (int e = shape_ok(N[i], K)) return e;
    if (!d_y[i] || !d_packed[i]) return W4A32_EINVAL;
    if (!aligned(d_packed[i], 16) || !aligned(d_y[i], 4)) return W4A32_EINVAL;
  }
  if (!aligned(d_x, 16) || !aligned(d_ws, 256)) return W4A32_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (count == 1) return w4a32_matmul(d_y[0], d_x, d_packed[0], d_ws, M, K, N[0], stream);
  if (w4::gemv_group_applies(M, K, N, count)) {
    const uint8_t* pk[W4A32_MAX_GROUP];
    for (int i = 0; i < count; ++i) pk[i] = static_cast<const uint8_t*>(d_packed[i]);
    return from_hip(w4::launch_gemv_group(d_y, d_x, K, pk, N, count, M, K, s));
  }
  // other sizes: quantise the rows once, then one launch of the f16 kernel over all the Linears
  // (M > 8) or one product per Linear
  if (int e = w4a32_quant_lhs(d_x, M, K, K, d_ws, stream)) return e;
  return w4a32_matmul_quantized_grouped(d_y, d_ws, d_packed, N, count, M, K, stream);
}

int w4a32_matmul_quantized_grouped(float* const* d_y, const void* d_ws, const void* const* d_packed,
                                   const int* N, int count, int M, int K, void* stream) {
  if (!d_y || !d_ws || !d_packed || !N) return W4A32_EINVAL;
  if (count < 1 || count > W4A32_MAX_GROUP || M <= 0) return W4A32_EINVAL;
  for (int i = 0; i < count; ++i) {
    if (int e = shape_ok(N[i], K)) return e;
    if (!d_y[i] || !d_packed[i]) return W4A32_EINVAL;
    if (!aligned(d_packed[i], 16) || !aligned(d_y[i], 4)) return W4A32_EINVAL;
  }
  if (!aligned(d_ws, 256)) return W4A32_EINVAL;
  if (M > w4::kGemvMaxM && count > 1) {
    const uint8_t* pk[W4A32_MAX_GROUP];
    for (int i = 0; i < count; ++i) pk[i] = static_cast<const uint8_t*>(d_packed[i]);
    return from_hip(w4::launch_gemm_group(d_y, static_cast<const uint8_t*>(d_ws), pk, N, count, M, K,
                                          static_cast<hipStream_t>(stream)));
  }
  for (int i = 0; i < count; ++i) {
    if (int e = w4a32_matmul_quantized(d_y[i], d_ws, d_packed[i], M, K, N[i], stream)) return e;
  }
  return W4A32_OK;
}

int w4a32_matmul_quantized_silu_pair(float* d_act, const void* d_ws, const void* d_gate, const void* d_up,
                                     int M, int K, int N, void* stream) {
  if (!d_act || !d_ws || !d_gate || !d_up || M <= 0) return W4A32_EINVAL;
  if (int e = shape_ok(N, K)) return e;
  if (M <= w4::kGemvMaxM) return W4A32_ESHAPE;  // the f16 product kernel's sizes only
  if (!aligned(d_ws, 256) || !aligned(d_gate, 16) || !aligned(d_up, 16) || !aligned(d_act, 4)) {
    return W4A32_EINVAL;
  }
  return from_hip(w4::launch_gemm_pair(d_act, static_cast<const uint8_t*>(d_ws),
                                       static_cast<const uint8_t*>(d_gate), static_cast<const uint8_t*>(d_up),
                                       M, K, N, static_cast<hipStream_t>(stream)));
}

}  // extern "C"
