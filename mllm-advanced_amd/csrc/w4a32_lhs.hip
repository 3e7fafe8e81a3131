// Per-row asymmetric int8 quantisation of the activations (runs in every forward).
//
// Bit-exact with the scalar model the reference's test holds
// (tests/Arm/KaiLinearTest.hpp:166-228): range always contains 0, scale = 255 / (rmax - rmin),
// the zero point is taken from the side with the smaller error, clamped, rounded to nearest
// even; values are round_half_away(x * scale) + zero_point, clamped to int8. Every f32 product
// and sum is an explicitly rounded intrinsic so no compiler flag can fuse them.
#include "w4a32_internal.h"
#include "w4a32_quant_math.h"

namespace w4 {

constexpr int kLhsThreads = 256;

// One workgroup per row. Pass 1 reads the row for min/max, pass 2 re-reads it (it is L2/L1
// resident: at most 35 KB) and writes 8 int8 per thread per step, plus the f16 copy of
// (a_q - zp), tiled in MFMA operand order, that the f16 MFMA prefill kernel consumes.
__global__ __launch_bounds__(kLhsThreads) void quant_lhs_kernel(
    const float* __restrict__ x, int K, int ldx, float* __restrict__ recip_out,
    int32_t* __restrict__ negzp_out, int8_t* __restrict__ aq, _Float16* __restrict__ ah) {
  const int m = blockIdx.x;
  const int t = threadIdx.x;
  const float* row = x + (size_t)m * ldx;

  float lo = 3.402823466e+38f, hi = -3.402823466e+38f;
  for (int i = 4 * t; i < K; i += 4 * kLhsThreads) {
    const float4 v = *reinterpret_cast<const float4*>(row + i);
    lo = fminf(fminf(lo, v.x), fminf(v.y, fminf(v.z, v.w)));
    hi = fmaxf(fmaxf(hi, v.x), fmaxf(v.y, fmaxf(v.z, v.w)));
  }
  lo = wave_minmax<false>(lo);
  hi = wave_minmax<true>(hi);
  __shared__ float s_lo[kLhsThreads / 64], s_hi[kLhsThreads / 64];
  if ((t & 63) == 0) {
    s_lo[t >> 6] = lo;
    s_hi[t >> 6] = hi;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kLhsThreads / 64; ++w) {
    lo = fminf(lo, s_lo[w]);
    hi = fmaxf(hi, s_hi[w]);
  }
  const RowQuant p = row_quant_params(lo, hi);
  const int zp = p.zp;

  if (t == 0) {
    recip_out[m] = p.recip;
    negzp_out[m] = -zp;
  }

  int8_t* dst = aq + (size_t)m * K;
  for (int i = 8 * t; i < K; i += 8 * kLhsThreads) {  // K % 32 == 0: whole groups of 8
    const float4 v0 = *reinterpret_cast<const float4*>(row + i);
    const float4 v1 = *reinterpret_cast<const float4*>(row + i + 4);
    const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
    int q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) q[e] = quant_one(f[e], p);
    uint2 packed;
    packed.x = pack4(q);
    packed.y = pack4(q + 4);
    *reinterpret_cast<uint2*>(dst + i) = packed;
    if (ah) {
      // a_q - zp lies in [-255, 255]: exact in f16. Stored in the order a weight dword unpacks.
      typedef _Float16 h8 __attribute__((ext_vector_type(8)));
      h8 hv;
#pragma unroll
      for (int e = 0; e < 8; ++e) hv[e] = (_Float16)(float)(q[kHalfOrder[e]] - zp);
      // chunk (m / 32, k-block) holds 32 rows x 32 k, 64 bytes per row (see w4a32_layout.h)
      const int kb = i >> 5, grp = (i >> 3) & 3;
      const size_t chunk = (size_t)(m >> 5) * (K >> 5) + kb;
      *reinterpret_cast<h8*>(ah + chunk * 1024 + (m & 31) * 32 + grp * 8) = hv;
    }
  }
}

// The same quantisation with the row held in registers (8 * R values per thread, K <= 2048 * R):
// one pass over memory, and room for what produces the row to run in front of it.
//   kSrcPlain:   row = a[m]                                   (row stride lda)
//   kSrcNorm:    s = a[m] (+ b[m]); h_out[m] = s;  row = s * (norm_w * 1/sqrt(mean(s^2) + eps))
//                (the residual add + RMSNorm that precedes q,k,v and gate,up; the f32 normalised
//                row is never written: only Linears read it)
//   kSrcSiluMul: row = a[m] / (1 + exp(-a[m])) * b[m]         (what down_proj reads)
// The element arithmetic is that of the standalone operators (rmsnorm_kernel, silu_mul_kernel);
// the sum of squares is accumulated in another order than rmsnorm_kernel's.
constexpr int kSrcPlain = 0, kSrcNorm = 1, kSrcSiluMul = 2;

template <int SRC, int R>
__global__ __launch_bounds__(kLhsThreads) void quant_rows_kernel(
    const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ norm_w,
    const float* __restrict__ part_bias, float eps, int K, int lda, int nparts, size_t part_stride,
    float* h_out,  // 16 dwords: preloaded by the dispatcher, everything the loads need; a read of the argument
                   // segment takes about half a microsecond
    float* __restrict__ recip_out, int32_t* __restrict__ negzp_out, int8_t* __restrict__ aq,
    _Float16* __restrict__ ah) {
  const int m = blockIdx.x;
  const int t = threadIdx.x;
  const size_t row = (size_t)m * lda;
  __shared__ float s_red[3][kLhsThreads / 64];

  float v[R][8];
  float ss = 0.0f;
  // the norm weights do not depend on the row: requested with it, not behind the sum of squares
  float4 g0[SRC == kSrcNorm ? R : 1], g1[SRC == kSrcNorm ? R : 1];
  if constexpr (SRC == kSrcNorm) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = 8 * t + 8 * kLhsThreads * r;
      const int ic = i < K ? i : 0;
      g0[r] = *reinterpret_cast<const float4*>(norm_w + ic);
      g1[r] = *reinterpret_cast<const float4*>(norm_w + ic + 4);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = 8 * t + 8 * kLhsThreads * r;
    if (i < K) {  // K % 32 == 0: whole groups of 8
      float4 x0 = *reinterpret_cast<const float4*>(a + row + i);
      float4 x1 = *reinterpret_cast<const float4*>(a + row + i + 4);
      if constexpr (SRC == kSrcNorm) {
        if (b) {
          float4 d0 = *reinterpret_cast<const float4*>(b + row + i);
          float4 d1 = *reinterpret_cast<const float4*>(b + row + i + 4);
          if (nparts > 0) {
            // b = the parts of a split-K product, [nparts][M][K] with the row and column factors applied:
            // delta = ((part 0 + part 1) + ...) + bias, clamped like every Linear output
            // four parts are requested at a time (one memory round trip, not four) and added in their order;
            // a part past the last one is read from part 0's place again and not added
            for (int p0 = 1; p0 < nparts; p0 += 4) {
              float4 e0[4], e1[4];
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const size_t off = (size_t)(p0 + q < nparts ? p0 + q : 0) * part_stride + row + i;
                e0[q] = *reinterpret_cast<const float4*>(b + off);
                e1[q] = *reinterpret_cast<const float4*>(b + off + 4);
              }
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                if (p0 + q < nparts) {
                  d0.x += e0[q].x; d0.y += e0[q].y; d0.z += e0[q].z; d0.w += e0[q].w;
                  d1.x += e1[q].x; d1.y += e1[q].y; d1.z += e1[q].z; d1.w += e1[q].w;
                }
              }
            }
            const float4 b0 = *reinterpret_cast<const float4*>(part_bias + i);
            const float4 b1 = *reinterpret_cast<const float4*>(part_bias + i + 4);
            constexpr float kMax = 3.402823466e+38f;
            d0.x = fminf(fmaxf(d0.x + b0.x, -kMax), kMax); d0.y = fminf(fmaxf(d0.y + b0.y, -kMax), kMax);
            d0.z = fminf(fmaxf(d0.z + b0.z, -kMax), kMax); d0.w = fminf(fmaxf(d0.w + b0.w, -kMax), kMax);
            d1.x = fminf(fmaxf(d1.x + b1.x, -kMax), kMax); d1.y = fminf(fmaxf(d1.y + b1.y, -kMax), kMax);
            d1.z = fminf(fmaxf(d1.z + b1.z, -kMax), kMax); d1.w = fminf(fmaxf(d1.w + b1.w, -kMax), kMax);
          }
          x0.x += d0.x; x0.y += d0.y; x0.z += d0.z; x0.w += d0.w;
          x1.x += d1.x; x1.y += d1.y; x1.z += d1.z; x1.w += d1.w;
          *reinterpret_cast<float4*>(h_out + row + i) = x0;
          *reinterpret_cast<float4*>(h_out + row + i + 4) = x1;
        }
        ss += x0.x * x0.x + x0.y * x0.y + x0.z * x0.z + x0.w * x0.w;
        ss += x1.x * x1.x + x1.y * x1.y + x1.z * x1.z + x1.w * x1.w;
      }
      if constexpr (SRC == kSrcSiluMul) {
        const float4 u0 = *reinterpret_cast<const float4*>(b + row + i);
        const float4 u1 = *reinterpret_cast<const float4*>(b + row + i + 4);
        x0.x = silu_mul(x0.x, u0.x);
        x0.y = silu_mul(x0.y, u0.y);
        x0.z = silu_mul(x0.z, u0.z);
        x0.w = silu_mul(x0.w, u0.w);
        x1.x = silu_mul(x1.x, u1.x);
        x1.y = silu_mul(x1.y, u1.y);
        x1.z = silu_mul(x1.z, u1.z);
        x1.w = silu_mul(x1.w, u1.w);
      }
      v[r][0] = x0.x; v[r][1] = x0.y; v[r][2] = x0.z; v[r][3] = x0.w;
      v[r][4] = x1.x; v[r][5] = x1.y; v[r][6] = x1.z; v[r][7] = x1.w;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[r][e] = 0.0f;  // the quantisation range always contains 0
    }
  }

  if constexpr (SRC == kSrcNorm) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if ((t & 63) == 0) s_red[2][t >> 6] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int w = 0; w < kLhsThreads / 64; ++w) tot += s_red[2][w];
    const float rstd = 1.0f / sqrtf(tot / (float)K + eps);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = 8 * t + 8 * kLhsThreads * r;
      if (i < K) {
        v[r][0] *= g0[r].x * rstd; v[r][1] *= g0[r].y * rstd; v[r][2] *= g0[r].z * rstd; v[r][3] *= g0[r].w * rstd;
        v[r][4] *= g1[r].x * rstd; v[r][5] *= g1[r].y * rstd; v[r][6] *= g1[r].z * rstd; v[r][7] *= g1[r].w * rstd;
      }
    }
  }

  float lo = 0.0f, hi = 0.0f;  // (min with 0, max with 0: what row_quant_params does anyway)
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      lo = fminf(lo, v[r][e]);
      hi = fmaxf(hi, v[r][e]);
    }
  lo = wave_minmax<false>(lo);
  hi = wave_minmax<true>(hi);
  if ((t & 63) == 0) {
    s_red[0][t >> 6] = lo;
    s_red[1][t >> 6] = hi;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kLhsThreads / 64; ++w) {
    lo = fminf(lo, s_red[0][w]);
    hi = fmaxf(hi, s_red[1][w]);
  }
  const RowQuant p = row_quant_params(lo, hi);
  const int zp = p.zp;
  if (t == 0) {
    recip_out[m] = p.recip;
    negzp_out[m] = -zp;
  }

  int8_t* dst = aq + (size_t)m * K;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = 8 * t + 8 * kLhsThreads * r;
    if (i >= K) continue;
    int q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) q[e] = quant_one(v[r][e], p);
    uint2 packed;
    packed.x = pack4(q);
    packed.y = pack4(q + 4);
    *reinterpret_cast<uint2*>(dst + i) = packed;
    if (ah) {
      typedef _Float16 h8 __attribute__((ext_vector_type(8)));
      h8 hv;
#pragma unroll
      for (int e = 0; e < 8; ++e) hv[e] = (_Float16)(float)(q[kHalfOrder[e]] - zp);
      const int kb = i >> 5, grp = (i >> 3) & 3;
      const size_t chunk = (size_t)(m >> 5) * (K >> 5) + kb;
      *reinterpret_cast<h8*>(ah + chunk * 1024 + (m & 31) * 32 + grp * 8) = hv;
    }
  }
}

// Largest K the register-resident kernel takes (8 values x 8 groups x 256 threads).
constexpr int kQuantRowsMaxK = 8 * 8 * kLhsThreads;

template <int SRC>
static hipError_t launch_quant_rows(const float* a, const float* b, const float* norm_w, float eps,
                                    float* h_out, int M, int K, int lda, uint8_t* ws, hipStream_t s,
                                    int nparts = 0, const float* part_bias = nullptr) {
  const WsGeom g = ws_geom(M, K);
  float* recip = reinterpret_cast<float*>(ws + g.scale_off);
  int32_t* negzp = reinterpret_cast<int32_t*>(ws + g.off_off);
  int8_t* aq = reinterpret_cast<int8_t*>(ws + g.aq_off);
  _Float16* ah = (M > kGemvMaxM) ? reinterpret_cast<_Float16*>(ws + g.ah_off) : nullptr;
  const int groups = (K + 8 * kLhsThreads - 1) / (8 * kLhsThreads);
#define W4_LAUNCH_ROWS(R)                                                                          \
  hipLaunchKernelGGL((quant_rows_kernel<SRC, R>), dim3(M), dim3(kLhsThreads), 0, s, a, b, norm_w,     \
                     part_bias, eps, K, lda, nparts, (size_t)M * K, h_out, recip, negzp, aq, ah)
  if (groups <= 1) W4_LAUNCH_ROWS(1);
  else if (groups <= 2) W4_LAUNCH_ROWS(2);
  else if (groups <= 5) W4_LAUNCH_ROWS(5);
  else if (groups <= 8) W4_LAUNCH_ROWS(8);
  else return hipErrorInvalidValue;
#undef W4_LAUNCH_ROWS
  return hipGetLastError();
}

bool quant_rows_fusable(int K) { return K <= kQuantRowsMaxK; }

hipError_t launch_quant_lhs_norm(const float* h, const float* delta, const float* norm_w, float eps,
                                 float* h_out, int M, int K, uint8_t* ws, hipStream_t s) {
  return launch_quant_rows<kSrcNorm>(h, delta, norm_w, eps, h_out, M, K, K, ws, s);
}

// The same with delta = the sum of a split-K product's `nparts` scaled parts ([nparts][M][K]) + bias.
hipError_t launch_quant_lhs_norm_parts(const float* h, const float* parts, int nparts, const float* bias,
                                       const float* norm_w, float eps, float* h_out, int M, int K,
                                       uint8_t* ws, hipStream_t s) {
  if (nparts < 1 || !parts || !bias) return hipErrorInvalidValue;
  return launch_quant_rows<kSrcNorm>(h, parts, norm_w, eps, h_out, M, K, K, ws, s, nparts, bias);
}

hipError_t launch_quant_lhs_silu_mul(const float* gate, const float* up, int M, int K, uint8_t* ws,
                                     hipStream_t s) {
  return launch_quant_rows<kSrcSiluMul>(gate, up, nullptr, 0.0f, nullptr, M, K, K, ws, s);
}

hipError_t launch_quant_lhs(const float* x, int M, int K, int ldx, uint8_t* ws, hipStream_t s) {
  if (K <= kQuantRowsMaxK) {
    return launch_quant_rows<kSrcPlain>(x, nullptr, nullptr, 0.0f, nullptr, M, K, ldx, ws, s);
  }
  const WsGeom g = ws_geom(M, K);
  float* recip = reinterpret_cast<float*>(ws + g.scale_off);
  int32_t* negzp = reinterpret_cast<int32_t*>(ws + g.off_off);
  int8_t* aq = reinterpret_cast<int8_t*>(ws + g.aq_off);
  _Float16* ah = (M > kGemvMaxM) ? reinterpret_cast<_Float16*>(ws + g.ah_off) : nullptr;
  hipLaunchKernelGGL(quant_lhs_kernel, dim3(M), dim3(kLhsThreads), 0, s, x, K, ldx, recip, negzp,
                     aq, ah);
  return hipGetLastError();
}

}  // namespace w4
