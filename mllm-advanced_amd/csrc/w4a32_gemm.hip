// Prefill product (M > 8): y[M][N] from quantised activation rows and the tiled 4-bit weights.
//
// Two kernels:
//
//  * gemm_f16_kernel (M > 32): v_mfma_f32_16x16x32_f16 on EXACT f16 operands. The activation
//    operand is a_q - zp (an integer in [-255, 255]); the weight operand is q * scale / 2^E_n
//    (4 + 8 significant bits), dequantised ONCE per workgroup from the 4-bit tiles into LDS,
//    already in MFMA fragment order. Every product is exact in f32; only the order of the f32
//    additions differs from the scalar model. No per-block work is left in the MFMA loop, which
//    is what lets the matrix cores run ahead of the VALU: with int8 MFMA every 32-k block would
//    need a convert + scale FMA per accumulator register, and that is VALU-bound.
//
//  * gemm_i8_kernel (9 <= M <= 32, and a cross-check for the other): integer path.
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

// ----------------------------------------------------------------------------------------
// f16 MFMA kernel
// ----------------------------------------------------------------------------------------

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

// 8 weights of one tile dword -> 8 f16 (q * s), in the order k0,k2,k4,k6,k1,k3,k5,k7.
// 0x6400 | u4 is the f16 number 1024 + u4; subtracting 1032 leaves q exactly.
__device__ __forceinline__ uint4 dequant8(uint32_t w, h2 s) {
  const uint32_t x = w ^ 0x88888888u;  // two's complement nibbles -> offset-8 nibbles
  uint32_t p[4];
  p[0] = (x & 0x000F000Fu) | 0x64006400u;
  p[1] = ((x >> 4) & 0x000F000Fu) | 0x64006400u;
  p[2] = ((x >> 8) & 0x000F000Fu) | 0x64006400u;
  p[3] = ((x >> 12) & 0x000F000Fu) | 0x64006400u;
  const h2 bias = {(_Float16)1032.0f, (_Float16)1032.0f};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    h2 v = __builtin_bit_cast(h2, p[i]);
    v = (v - bias) * s;
    o[i] = __builtin_bit_cast(uint32_t, v);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

constexpr int kF16BK = 64;  // k per LDS stage (two scale blocks, half of a weight tile chunk)

// Workgroup = 4 wavefronts arranged 2 (M) x 2 (N) over a BM x BN output tile.
// LDS holds one stage: A as [2 k-blocks][BM/16 fragments][16 rows][32 k] f16 and B likewise;
// a fragment is 1 KiB contiguous, and lane (g, j) reads its 16 bytes at j*64 + g*16.
// The next stage travels global -> registers while the current one is multiplied.
template <int BM, int BN>
__global__ __launch_bounds__(256, 2) void gemm_f16_kernel(
    float* __restrict__ y, const _Float16* __restrict__ ah, const float* __restrict__ recip,
    const uint8_t* __restrict__ packed, const uint8_t* __restrict__ hscale,
    const float* __restrict__ rowmul, const float* __restrict__ bias, int M, int N, int K, int NT,
    int KC) {
  constexpr int MT = BM / 16, NTW = BN / 16;
  constexpr int WMT = MT / 2, WNT = NTW / 2;
  constexpr int A_UNITS = BM * 8 / 256;    // 16-byte pieces of A per thread per stage
  constexpr int B_UNITS = NTW * 64 / 256;  // 8-byte pieces of packed B per thread per stage
  static_assert(B_UNITS >= 1, "BN too small");

  __shared__ __align__(16) uint8_t lds[(BM + BN) * kF16BK * 2];
  uint8_t* sA = lds;
  uint8_t* sB = lds + BM * kF16BK * 2;

  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int g = lane >> 4, j = lane & 15;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM;
  const int nt0 = blockIdx.x * NTW;

  uint4 ra[A_UNITS];
  uint2 rb[B_UNITS];
  uint32_t rs[B_UNITS];

  auto load_stage = [&](int s) {
    const int k0 = s * kF16BK;
#pragma unroll
    for (int u = 0; u < A_UNITS; ++u) {
      const int unit = t + 256 * u;
      const int row = unit >> 3, kseg = unit & 7;
      int gr = m0 + row;
      gr = gr < M ? gr : M - 1;  // rows past M repeat the last row; their outputs are not stored
      const int kk = k0 + 8 * kseg;
      ra[u] = make_uint4(0, 0, 0, 0);
      if (kk < K) ra[u] = *reinterpret_cast<const uint4*>(ah + (size_t)gr * K + kk);
    }
    const int kc = s >> 1, half = s & 1;
#pragma unroll
    for (int u = 0; u < B_UNITS; ++u) {
      const int unit = t + 256 * u;
      const int ntl = unit >> 6, ln = unit & 63;
      const int nt = nt0 + ntl;
      rb[u] = make_uint2(0, 0);
      rs[u] = 0;
      if (nt < NT) {
        const size_t tile = (size_t)nt * KC + kc;
        rb[u] = *reinterpret_cast<const uint2*>(packed + tile * kTileBytes + 16 * ln + 8 * half);
        rs[u] = *reinterpret_cast<const uint32_t*>(hscale + tile * kTileScaleBytes + 8 * (ln & 15) +
                                                   4 * half);
      }
    }
  };

  auto store_stage = [&]() {
#pragma unroll
    for (int u = 0; u < A_UNITS; ++u) {
      const int unit = t + 256 * u;
      const int row = unit >> 3, kseg = unit & 7;
      const int kb = kseg >> 2, gg = kseg & 3;
      const int off = (((kb * MT + (row >> 4)) * 16 + (row & 15)) * 64) + gg * 16;
      *reinterpret_cast<uint4*>(sA + off) = ra[u];
    }
#pragma unroll
    for (int u = 0; u < B_UNITS; ++u) {
      const int unit = t + 256 * u;
      const int ntl = unit >> 6, ln = unit & 63;
      const int lane_off = (ln & 15) * 64 + (ln >> 4) * 16;
      const h2 s2 = __builtin_bit_cast(h2, rs[u]);
      const h2 s_lo = {s2[0], s2[0]};
      const h2 s_hi = {s2[1], s2[1]};
      *reinterpret_cast<uint4*>(sB + (0 * NTW + ntl) * 1024 + lane_off) = dequant8(rb[u].x, s_lo);
      *reinterpret_cast<uint4*>(sB + (1 * NTW + ntl) * 1024 + lane_off) = dequant8(rb[u].y, s_hi);
    }
  };

  v4f acc[WMT][WNT];
#pragma unroll
  for (int a = 0; a < WMT; ++a)
#pragma unroll
    for (int b = 0; b < WNT; ++b) acc[a][b] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

  const int nstages = (K + kF16BK - 1) / kF16BK;
  const int frag_off = j * 64 + g * 16;
  load_stage(0);
  for (int s = 0; s < nstages; ++s) {
    __syncthreads();  // every wavefront has finished reading the previous stage
    store_stage();
    __syncthreads();
    if (s + 1 < nstages) load_stage(s + 1);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      h8 af[WMT], bf[WNT];
#pragma unroll
      for (int a = 0; a < WMT; ++a)
        af[a] = *reinterpret_cast<const h8*>(sA + (kb * MT + wm * WMT + a) * 1024 + frag_off);
#pragma unroll
      for (int b = 0; b < WNT; ++b)
        bf[b] = *reinterpret_cast<const h8*>(sB + (kb * NTW + wn * WNT + b) * 1024 + frag_off);
#pragma unroll
      for (int a = 0; a < WMT; ++a)
#pragma unroll
        for (int b = 0; b < WNT; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[a], bf[b], acc[a][b], 0, 0, 0);
    }
  }

  // C layout: lane (g, j) holds column j, rows 4*g + r of each 16x16 tile.
#pragma unroll
  for (int b = 0; b < WNT; ++b) {
    const int n = 16 * (nt0 + wn * WNT + b) + j;
    if (n >= N) continue;
    const float rm = rowmul[n], bs = bias[n];
#pragma unroll
    for (int a = 0; a < WMT; ++a) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + 16 * (wm * WMT + a) + 4 * g + r;
        if (m < M) {
          float v = acc[a][b][r] * rm;
          v = __fmaf_rn(v, recip[m], bs);
          v = fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
          y[(size_t)m * N + n] = v;
        }
      }
    }
  }
}

template <int BM, int BN>
static hipError_t launch_f16(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                             hipStream_t s) {
  const WeightGeom g = weight_geom(N, K);
  const WsGeom w = ws_geom(M, K);
  dim3 grid((g.NT + BN / 16 - 1) / (BN / 16), (M + BM - 1) / BM);
  hipLaunchKernelGGL((gemm_f16_kernel<BM, BN>), grid, dim3(256), 0, s, y,
                     reinterpret_cast<const _Float16*>(ws + w.ah_off),
                     reinterpret_cast<const float*>(ws + w.scale_off), packed,
                     packed + g.hscale_off, reinterpret_cast<const float*>(packed + g.rowmul_off),
                     reinterpret_cast<const float*>(packed + g.bias_off), M, N, K, g.NT, g.KC);
  return hipGetLastError();
}

static hipError_t launch_gemm_i8(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K,
                                 int N, hipStream_t s) {
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

// Tile choice: the chip has 256 CUs with two workgroups resident each. Prefer the largest tile
// that still yields enough workgroups; a tile with a larger wavefront tile reuses each LDS
// fragment more often, so it is weighted up.
static int pick_f16_tile(int M, int NT) {
  struct Cand { int bm, bn; double w; };
  const Cand cands[3] = {{256, 128, 1.0}, {128, 128, 0.8}, {128, 64, 0.6}};
  const double slots = 512.0;
  int best = 0;
  double best_score = -1.0;
  for (int i = 0; i < 3; ++i) {
    const long tiles = (long)((M + cands[i].bm - 1) / cands[i].bm) *
                       ((NT + cands[i].bn / 16 - 1) / (cands[i].bn / 16));
    const double rounds = (double)((tiles + (long)slots - 1) / (long)slots);
    const double useful = ((double)M * NT * 16) / ((double)tiles * cands[i].bm * cands[i].bn);
    const double score = cands[i].w * useful * (double)tiles / (rounds * slots);
    if (score > best_score) {
      best_score = score;
      best = i;
    }
  }
  return best;
}

hipError_t launch_gemm(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                       int kernel, hipStream_t s) {
  if (kernel == kKernelGemmI8 || (kernel == kKernelAuto && M <= 32)) {
    return launch_gemm_i8(y, ws, packed, M, K, N, s);
  }
  const WeightGeom g = weight_geom(N, K);
  switch (pick_f16_tile(M, g.NT)) {
    case 0: return launch_f16<256, 128>(y, ws, packed, M, K, N, s);
    case 1: return launch_f16<128, 128>(y, ws, packed, M, K, N, s);
    default: return launch_f16<128, 64>(y, ws, packed, M, K, N, s);
  }
}

}  // namespace w4
