// Dense (unquantised) [N][K] operands held as f16 or f32, for the parameters the reference's W4A32 quantizer
// leaves unquantised: lm_head, which the model applies as a plain matmul with transpose_b
// (mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:209-213, kept Fp16 by scripts/QuantCfg/ds_qwen2/1.5B-W4A32-KAI.json:43-45),
// and the norm weights (Fp16 in the same file, :33-42), which are widened to f32 once at load.
//
//   f16_to_f32_kernel   n halves -> n floats (exact)
//   dense_rows_kernel   C[m][n] = sum_k A[m][k] B[n][k] for M <= 8 rows of A: a stream over B, read once.
//                       HBM-bound: N * K * sizeof(B element) bytes.
//
// dense_rows_kernel: the M rows of A sit in LDS as f32; 16 lanes share a row of B, a wavefront takes four rows
// at a time. Lane j of a row's 16 multiplies k = 128 i + 8 j + 0..7 for i = 0, 1, ... (one 16-byte load of
// f16, two of f32), sums its products in that order with one FMA each, and the 16 partial sums meet in four DPP
// steps. An f16 element widens to f32 exactly, so the f16 and the f32 form of the same values give the same
// bits. At M = 1 the kernel can complete and normalise the row first (residual add of up to three partial rows
// + RMSNorm, as the decoder's step needs in front of lm_head) and leave one (largest output, its first column)
// pair per wavefront for a greedy sampler.
#include <algorithm>

#include "w4a32_decoder.h"
#include "w4a32_internal.h"
#include "w4a32_quant_math.h"

namespace w4 {

namespace {

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));

__global__ __launch_bounds__(256) void f16_to_f32_kernel(const _Float16* __restrict__ in, float* __restrict__ out,
                                                         size_t n, int vec_ok) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t n8 = vec_ok ? n / 8 : 0;
  for (size_t v = i; v < n8; v += stride) {
    const h8_t h = *reinterpret_cast<const h8_t*>(in + 8 * v);
    reinterpret_cast<float4*>(out + 8 * v)[0] = make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
    reinterpret_cast<float4*>(out + 8 * v)[1] = make_float4((float)h[4], (float)h[5], (float)h[6], (float)h[7]);
  }
  for (size_t e = 8 * n8 + i; e < n; e += stride) out[e] = (float)in[e];
}

// eight consecutive elements of a row of B, as they come from memory
template <typename WT>
struct Raw8;
template <>
struct Raw8<_Float16> {
  h8_t v;
  __device__ __forceinline__ void load(const _Float16* p) { v = *reinterpret_cast<const h8_t*>(p); }
  __device__ __forceinline__ float get(int e) const { return (float)v[e]; }
};
template <>
struct Raw8<float> {
  float4 a, b;
  __device__ __forceinline__ void load(const float* p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  __device__ __forceinline__ float get(int e) const {
    const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    return f[e];
  }
};

constexpr int kDenseWaves = 4;   // wavefronts per workgroup
constexpr int kDenseBatch = 4;   // 8-element loads a lane keeps in flight per batch (two batches at a time)

struct DenseRowPrologue {
  const float* delta;   // optional, M = 1: added to the row first; delta_parts rows, K floats apart
  int delta_parts;
  const float* norm_w;  // RMSNorm weight [K]
  float eps;
  float* amax_val;      // optional, M = 1: per wavefront of the launch, the largest output it stored ...
  int* amax_idx;        // ... and its first column (-inf and 0x7fffffff when it stored none)
};

template <typename WT, int M, bool kNorm>
__global__ __launch_bounds__(64 * kDenseWaves) void dense_rows_kernel(const float* __restrict__ x, int ldx,
                                                                      const WT* __restrict__ b,
                                                                      float* __restrict__ c, int N, int K, int KI,
                                                                      const DenseRowPrologue pro) {
  extern __shared__ __align__(16) float s_x[];  // [M][Kp], zeros past K
  __shared__ float s_part[kDenseWaves];
  const int Kp = KI * 128;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 4, j = lane & 15;

  if constexpr (kNorm) {
    static_assert(M == 1, "the norm prologue serves one row");
    float ss = 0.0f;
    for (int i = 4 * threadIdx.x; i < Kp; i += 4 * 64 * kDenseWaves) {
      float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (i < K) {
        v = *reinterpret_cast<const float4*>(x + i);
        if (pro.delta) {
          float4 d = *reinterpret_cast<const float4*>(pro.delta + i);
          for (int p = 1; p < pro.delta_parts; ++p) {  // ((r0 + r1) + r2), as the W4A32 kernels add partial rows
            const float4 e = *reinterpret_cast<const float4*>(pro.delta + (size_t)p * K + i);
            d.x += e.x; d.y += e.y; d.z += e.z; d.w += e.w;
          }
          if (pro.delta_parts > 1) {  // the parts' sum is a Linear's output: clamped like every other one
            d.x = fminf(fmaxf(d.x, -3.402823466e+38f), 3.402823466e+38f);
            d.y = fminf(fmaxf(d.y, -3.402823466e+38f), 3.402823466e+38f);
            d.z = fminf(fmaxf(d.z, -3.402823466e+38f), 3.402823466e+38f);
            d.w = fminf(fmaxf(d.w, -3.402823466e+38f), 3.402823466e+38f);
          }
          v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      }
      *reinterpret_cast<float4*>(s_x + i) = v;
    }
    ss = wave_sum_to_lane63(ss);
    if (lane == 63) s_part[wave] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kDenseWaves; ++w) total += s_part[w];
    const float rstd = 1.0f / sqrtf(total / (float)K + pro.eps);
    for (int i = 4 * threadIdx.x; i < K; i += 4 * 64 * kDenseWaves) {  // the elements this thread wrote
      const float4 w = *reinterpret_cast<const float4*>(pro.norm_w + i);
      float4 v = *reinterpret_cast<float4*>(s_x + i);
      v.x = v.x * (w.x * rstd); v.y = v.y * (w.y * rstd); v.z = v.z * (w.z * rstd); v.w = v.w * (w.w * rstd);
      *reinterpret_cast<float4*>(s_x + i) = v;
    }
  } else {
    for (int i = 4 * threadIdx.x; i < M * Kp; i += 4 * 64 * kDenseWaves) {
      const int m = i / Kp, k = i - m * Kp;
      float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (k < K) v = *reinterpret_cast<const float4*>(x + (size_t)m * ldx + k);
      *reinterpret_cast<float4*>(s_x + i) = v;
    }
  }
  __syncthreads();

  const int gw = (int)blockIdx.x * kDenseWaves + wave, nw = (int)gridDim.x * kDenseWaves;
  const int RG = (N + 3) / 4;                          // groups of four rows of B
  const int NB = (KI + kDenseBatch - 1) / kDenseBatch;  // batches per row
  // batch bt of row group rg: loads i = bt * kDenseBatch .. + kDenseBatch - 1; past K the address is the row's
  // start and the value is not used
  auto load_batch = [&](int rg, int bt, Raw8<WT> (&raw)[kDenseBatch]) {
    const int n = 4 * rg + g;
    const WT* row = b + (size_t)(n < N ? n : N - 1) * K;
#pragma unroll
    for (int u = 0; u < kDenseBatch; ++u) {
      const int k = 128 * (bt * kDenseBatch + u) + 8 * j;
      raw[u].load(row + (k < K ? k : 0));
    }
  };
  float best_v = -INFINITY;
  int best_n = 0x7fffffff;
  Raw8<WT> cur[kDenseBatch];
  if (gw < RG) load_batch(gw, 0, cur);
  for (int rg = gw; rg < RG; rg += nw) {
    float acc[M];
#pragma unroll
    for (int m = 0; m < M; ++m) acc[m] = 0.0f;
    for (int bt = 0; bt < NB; ++bt) {
      // request the next batch (of this row group, or the first of this wavefront's next one), then multiply
      Raw8<WT> nxt[kDenseBatch];
      const bool last = bt + 1 == NB;
      const int rg_n = last ? rg + nw : rg, bt_n = last ? 0 : bt + 1;
      if (rg_n < RG) {
        load_batch(rg_n, bt_n, nxt);
      } else {
#pragma unroll
        for (int u = 0; u < kDenseBatch; ++u) nxt[u] = cur[u];
      }
#pragma unroll
      for (int u = 0; u < kDenseBatch; ++u) {
        const int k = 128 * (bt * kDenseBatch + u) + 8 * j;
        if (k < K) {
#pragma unroll
          for (int m = 0; m < M; ++m) {
            const float4 x0 = *reinterpret_cast<const float4*>(s_x + (size_t)m * Kp + k);
            const float4 x1 = *reinterpret_cast<const float4*>(s_x + (size_t)m * Kp + k + 4);
            const float xs[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[m] = __fmaf_rn(cur[u].get(e), xs[e], acc[m]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kDenseBatch; ++u) cur[u] = nxt[u];
    }
    const int n = 4 * rg + g;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float t = row16_sum_all(acc[m]);
      if (j == 0 && n < N) {
        c[(size_t)m * N + n] = t;
        if (M == 1 && (t > best_v || (t == best_v && n < best_n))) {
          best_v = t;
          best_n = n;
        }
      }
    }
  }
  if constexpr (M == 1) {
    if (pro.amax_val) {
      // lanes 0, 16, 32, 48 hold the candidates of their rows: the largest value, the lowest column among equals
#pragma unroll
      for (int off = 32; off >= 16; off >>= 1) {
        const float ov = __shfl_xor(best_v, off, 64);
        const int on = __shfl_xor(best_n, off, 64);
        if (ov > best_v || (ov == best_v && on < best_n)) {
          best_v = ov;
          best_n = on;
        }
      }
      if (lane == 0) {
        pro.amax_val[gw] = best_v;
        pro.amax_idx[gw] = best_n;
      }
    }
  }
}

int dense_grid(int N) {
  const int RG = (N + 3) / 4;
  return std::min((RG + kDenseWaves - 1) / kDenseWaves, 1024);
}

template <typename WT, int M, bool kNorm>
hipError_t launch_dense_rows_m(const float* x, int ldx, const void* b, float* c, int N, int K,
                               const DenseRowPrologue& pro, hipStream_t s) {
  const int KI = (K + 127) / 128;
  const size_t lds = (size_t)M * KI * 128 * sizeof(float);
  auto kern = dense_rows_kernel<WT, M, kNorm>;
  static LdsLimitOnce raised;
  if (lds > 64 * 1024) {
    if (hipError_t e = raised.raise(reinterpret_cast<const void*>(kern), 160 * 1024); e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3(dense_grid(N)), dim3(64 * kDenseWaves), lds, s, x, ldx, static_cast<const WT*>(b), c,
                     N, K, KI, pro);
  return hipGetLastError();
}

template <typename WT>
hipError_t launch_dense_rows_t(const float* x, int ldx, const void* b, float* c, int M, int N, int K,
                               hipStream_t s) {
  const DenseRowPrologue none{nullptr, 0, nullptr, 0.0f, nullptr, nullptr};
  switch (M) {
    case 1: return launch_dense_rows_m<WT, 1, false>(x, ldx, b, c, N, K, none, s);
    case 2: return launch_dense_rows_m<WT, 2, false>(x, ldx, b, c, N, K, none, s);
    case 3: return launch_dense_rows_m<WT, 3, false>(x, ldx, b, c, N, K, none, s);
    case 4: return launch_dense_rows_m<WT, 4, false>(x, ldx, b, c, N, K, none, s);
    case 5: return launch_dense_rows_m<WT, 5, false>(x, ldx, b, c, N, K, none, s);
    case 6: return launch_dense_rows_m<WT, 6, false>(x, ldx, b, c, N, K, none, s);
    case 7: return launch_dense_rows_m<WT, 7, false>(x, ldx, b, c, N, K, none, s);
    case 8: return launch_dense_rows_m<WT, 8, false>(x, ldx, b, c, N, K, none, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

hipError_t launch_f16_to_f32(const void* in, float* out, size_t n, hipStream_t s) {
  const int vec_ok = (reinterpret_cast<uintptr_t>(in) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  const size_t want = (n / 8 + 255) / 256 + 1;
  hipLaunchKernelGGL(f16_to_f32_kernel, dim3((unsigned)std::min<size_t>(want, 4096)), dim3(256), 0, s,
                     static_cast<const _Float16*>(in), out, n, vec_ok);
  return hipGetLastError();
}

bool dense_rows_applies(int M, int K) {
  // K in whole 8-element loads, and the M rows (padded to 128) fit the LDS
  return M >= 1 && M <= 8 && K > 0 && K % 8 == 0 && (size_t)M * ((K + 127) / 128) * 512 <= 160 * 1024;
}

int dense_rows_partials(int N) { return dense_grid(N) * kDenseWaves; }

hipError_t launch_dense_rows(const float* x, int ldx, const void* b, int b_dtype, float* c, int M, int N, int K,
                             hipStream_t s) {
  if (!dense_rows_applies(M, K)) return hipErrorInvalidValue;
  if (b_dtype == W4A32_DENSE_F16) return launch_dense_rows_t<_Float16>(x, ldx, b, c, M, N, K, s);
  if (b_dtype == W4A32_DENSE_F32) return launch_dense_rows_t<float>(x, ldx, b, c, M, N, K, s);
  return hipErrorInvalidValue;
}

hipError_t launch_dense_head(const float* h, const float* delta, int delta_parts, const float* norm_w, float eps,
                             const void* b, int b_dtype, float* logits, int N, int K, float* amax_val,
                             int* amax_idx, hipStream_t s) {
  if (!dense_rows_applies(1, K) || !norm_w) return hipErrorInvalidValue;
  const DenseRowPrologue pro{delta, delta ? std::max(delta_parts, 1) : 0, norm_w, eps, amax_val, amax_idx};
  if (b_dtype == W4A32_DENSE_F16) return launch_dense_rows_m<_Float16, 1, true>(h, K, b, logits, N, K, pro, s);
  if (b_dtype == W4A32_DENSE_F32) return launch_dense_rows_m<float, 1, true>(h, K, b, logits, N, K, pro, s);
  return hipErrorInvalidValue;
}

}  // namespace w4
