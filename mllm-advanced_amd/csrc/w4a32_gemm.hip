// Prefill product (M > 8): y[M][N] from quantised activation rows and the tiled 4-bit weights.
//
// Integer path: v_mfma_i32_16x16x32_i8. One MFMA spans exactly one scale block (32 k), so the
// block sums are exact int32, as in the reference's scalar model
// (tests/Arm/KaiLinearTest.hpp:342-372); each is converted and scaled in f32 by the block's
// scale. A wavefront owns one 16-row weight tile row and a 64-row slab of activations:
// dword d of its 128-bit weight load is directly the B operand (two mask ops), the A operand
// is 8 consecutive int8 of an activation row.
#include "w4a32_internal.h"

namespace w4 {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kGemmI8MTiles = 4;   // 16-row activation tiles per wavefront
constexpr int kGemmI8Waves = 4;    // weight tile rows per workgroup

__global__ __launch_bounds__(64 * kGemmI8Waves) void gemm_i8_kernel(
    float* __restrict__ y, const int8_t* __restrict__ aq, const float* __restrict__ recip,
    const int32_t* __restrict__ negzp, const uint8_t* __restrict__ packed, int M, int Mp, int N,
    int K, int NT, int KC, const float* __restrict__ rsum, const float* __restrict__ bias) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 4, j = lane & 15;
  const int nt = blockIdx.x * kGemmI8Waves + wave;
  const int m0 = blockIdx.y * 16 * kGemmI8MTiles;
  if (nt >= NT) return;

  const uint8_t* tiles = packed + (size_t)nt * KC * kTileBytes;

  // A rows this lane feeds (row = lane % 16 of each 16-row tile); rows past Mp-1 are clamped,
  // their products land in output rows that are never stored.
  const int8_t* a_row[kGemmI8MTiles];
#pragma unroll
  for (int mt = 0; mt < kGemmI8MTiles; ++mt) {
    int r = m0 + 16 * mt + j;
    r = r < Mp ? r : Mp - 1;
    a_row[mt] = aq + (size_t)r * K + 8 * g;
  }

  float acc[kGemmI8MTiles][4];
#pragma unroll
  for (int mt = 0; mt < kGemmI8MTiles; ++mt)
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[mt][r] = 0.0f;

  for (int kc = 0; kc < KC; ++kc) {
    const uint4 wq = *reinterpret_cast<const uint4*>(tiles + (size_t)kc * kTileBytes + 16 * lane);
    const uint2 sc =
        *reinterpret_cast<const uint2*>(tiles + (size_t)kc * kTileBytes + kTileQBytes + 8 * j);
    const uint32_t wv[4] = {wq.x, wq.y, wq.z, wq.w};
    const float sv[4] = {__uint_as_float(sc.x << 16), __uint_as_float(sc.x & 0xFFFF0000u),
                         __uint_as_float(sc.y << 16), __uint_as_float(sc.y & 0xFFFF0000u)};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int kk = kTileK * kc + kBlockLen * d;
      if (kk >= K) break;  // chunk padding (uniform across the wavefront)
      const uint32_t lo = (wv[d] << 4) & 0xF0F0F0F0u;
      const uint32_t hi = wv[d] & 0xF0F0F0F0u;
      const long b64 = (long)(((unsigned long)hi << 32) | lo);
#pragma unroll
      for (int mt = 0; mt < kGemmI8MTiles; ++mt) {
        const long a64 = *reinterpret_cast<const long*>(a_row[mt] + kk);
        v4i c = {0, 0, 0, 0};
        c = __builtin_amdgcn_mfma_i32_16x16x32_i8(a64, b64, c, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[mt][r] = __fmaf_rn((float)c[r], sv[d], acc[mt][r]);
      }
    }
  }

  // C layout: lane (g, j) holds column j, rows 4*g + r.
  const int n = kTileRows * nt + j;
  if (n >= N) return;
  const float rs = rsum[n], bs = bias[n];
#pragma unroll
  for (int mt = 0; mt < kGemmI8MTiles; ++mt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + 16 * mt + 4 * g + r;
      if (m < M) {
        float v = __fmaf_rn((float)negzp[m], rs, acc[mt][r] * 0.0625f);
        v = __fmaf_rn(v, recip[m], bs);
        v = fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
        y[(size_t)m * N + n] = v;
      }
    }
  }
}

hipError_t launch_gemm(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                       hipStream_t s) {
  const WeightGeom g = weight_geom(N, K);
  const WsGeom w = ws_geom(M, K);
  dim3 grid((g.NT + kGemmI8Waves - 1) / kGemmI8Waves,
            (M + 16 * kGemmI8MTiles - 1) / (16 * kGemmI8MTiles));
  hipLaunchKernelGGL(gemm_i8_kernel, grid, dim3(64 * kGemmI8Waves), 0, s, y,
                     reinterpret_cast<const int8_t*>(ws + w.aq_off),
                     reinterpret_cast<const float*>(ws + w.scale_off),
                     reinterpret_cast<const int32_t*>(ws + w.off_off), packed, M, w.Mp, N, K, g.NT,
                     g.KC, reinterpret_cast<const float*>(packed + g.rsum_off),
                     reinterpret_cast<const float*>(packed + g.bias_off));
  return hipGetLastError();
}

}  // namespace w4
