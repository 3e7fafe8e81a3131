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

hipError_t launch_quant_lhs(const float* x, int M, int K, int ldx, uint8_t* ws, hipStream_t s) {
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
