// Prefill product (M > 8): y[M][N] from quantised activation rows and the tiled 4-bit weights.
//
// Two kernels:
//
//  * gemm_f16_kernel (M > 32): v_mfma_f32_32x32x16_f16 on EXACT f16 operands. The activation
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
// 0x6400 | u4 is the f16 number 1024 + u4, and 0x6400 | (u4 << 4) is 1024 + 16*u4, so the
// nibbles at bits 0-3 and 4-7 of each half-word need no shift: subtract 1032 (resp. 1152) to
// get q (resp. 16*q) exactly, then multiply by s (resp. s/16). `s` holds {s, s} and `s16`
// holds {s/16, s/16}; s/16 is exact unless s is already a subnormal f16.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t m, uint32_t o) {
  return (a & m) | o;  // one v_and_or_b32
}
__device__ __forceinline__ uint4 dequant8(uint32_t w, h2 s, h2 s16) {
  const uint32_t x = w ^ 0x88888888u;  // two's complement nibbles -> offset-8 nibbles
  const uint32_t xh = x >> 8;
  const h2 b1 = {(_Float16)1032.0f, (_Float16)1032.0f};
  const h2 b16 = {(_Float16)1152.0f, (_Float16)1152.0f};
  const h2 p0 = __builtin_bit_cast(h2, and_or(x, 0x000F000Fu, 0x64006400u));   // nibbles 0,4
  const h2 p1 = __builtin_bit_cast(h2, and_or(x, 0x00F000F0u, 0x64006400u));   // nibbles 1,5
  const h2 p2 = __builtin_bit_cast(h2, and_or(xh, 0x000F000Fu, 0x64006400u));  // nibbles 2,6
  const h2 p3 = __builtin_bit_cast(h2, and_or(xh, 0x00F000F0u, 0x64006400u));  // nibbles 3,7
  const h2 o0 = (p0 - b1) * s;
  const h2 o1 = (p1 - b16) * s16;
  const h2 o2 = (p2 - b1) * s;
  const h2 o3 = (p3 - b16) * s16;
  return make_uint4(__builtin_bit_cast(uint32_t, o0), __builtin_bit_cast(uint32_t, o1),
                    __builtin_bit_cast(uint32_t, o2), __builtin_bit_cast(uint32_t, o3));
}

constexpr int kF16BK = 64;    // k per stage (two scale blocks, half of a weight tile chunk)

typedef float v16f __attribute__((ext_vector_type(16)));

// v_mfma_f32_32x32x16_f16 (measured on MI355X: 2.1-2.2 PFLOP/s, twice the 16x16x32 shape).
// Operands: lane l = 32*h + i holds 8 f16 of row/column i at "k-slot" h. Which k values a slot
// stands for is free as long as A and B agree; here, inside a 32-k scale block, slice 0 is
// k {0..7 | 16..23} for h = {0 | 1} and slice 1 is k {8..15 | 24..31}, so that one lane's two A
// operands of a block are 32 contiguous bytes of its activation row.
//
// Workgroup = 4 wavefronts stacked along M; wavefront w owns rows [32*WM*w, 32*WM*(w+1)) of
// the BM x BN tile (BM = 128*WM, BN = 32*WN) and all BN columns.
//
//  * A (f16 activations) never touches LDS: the row quantiser already wrote it as 2 KiB chunks
//    of 32 rows x 32 k, so the two operand loads of a block read one contiguous chunk (instead
//    of 32 rows that lie K*2 bytes apart), into a register ring DEPTH stages deep (a load
//    has that many stages of MFMA work to land).
//  * B (4-bit weights) is shared by the four wavefronts: its packed bytes are prefetched into
//    a small register ring, dequantised once per workgroup to f16 and double-buffered in LDS
//    as 1 KiB fragments in lane order (lane l at l*16: conflict-free 128-bit accesses).
//  * One barrier per stage: it publishes the B buffer written during the previous stage and
//    frees the one read during it.
// DEPTH = stages between a global load and its use: 2 for the large tiles (registers), 4 for the
// small ones, whose stages are short next to the memory latency.
template <int WAVES_M, int WAVES_N, int WM, int WN, int DEPTH>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_f16_kernel(
    float* __restrict__ y, const _Float16* __restrict__ ah, const float* __restrict__ recip,
    const uint8_t* __restrict__ packed, const uint8_t* __restrict__ hscale,
    const float* __restrict__ rowmul, const float* __restrict__ bias, int M, int N, int K, int NT,
    int KC, int MB, int NB, int n_major) {
  constexpr int D = DEPTH;
  static_assert(D % 2 == 0, "stage s uses LDS buffer s & 1: the unrolled ring must keep that parity");
  constexpr int NWAVES = WAVES_M * WAVES_N;
  constexpr int BM = 32 * WM * WAVES_M;
  constexpr int BN32 = WN * WAVES_N;           // 32-column fragments per workgroup and k-slice
  constexpr int WNT = 2 * BN32;                // 16-row weight tile rows per workgroup
  static_assert(WNT % NWAVES == 0, "each wavefront dequantises WNT/NWAVES tile rows per stage");
  constexpr int B_UNITS = WNT / NWAVES;        // 8-byte pieces of packed B per thread per stage
  constexpr int kBufBytes = 4 * BN32 * 1024;   // one B stage: [4 k-slices][BN32 fragments]

  __shared__ __align__(16) uint8_t sB[2 * kBufBytes];

  const int t = threadIdx.x;
  const int wave = t >> 6, lane = t & 63;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int g = lane >> 4, j = lane & 15;     // position inside a weight tile
  const int h = lane >> 5, i32 = lane & 31;   // position inside an MFMA operand / C tile
  // Workgroup -> tile. The hardware deals consecutive workgroups round-robin to the 8 XCDs, each
  // with its own L2. Workgroup b therefore takes tile (b % 8) * ceil(T / 8) + b / 8, so that an
  // XCD owns one contiguous run of tiles; the run is ordered so that neighbours share the larger
  // operand (n_major: all row blocks of a weight column block together, weights fetched by one
  // XCD only; otherwise all column blocks of a row block together).
  const int total = MB * NB;
  const int per_xcd = (total + 7) >> 3;
  const int tile = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
  if (tile >= total) return;  // whole workgroup: no barrier has been reached yet
  const int mb = n_major ? tile % MB : tile / NB;
  const int nb = n_major ? tile / MB : tile % NB;
  const int m0 = mb * BM + 32 * WM * wm;
  const int nt0 = nb * WNT;
  const int nstages = (K + kF16BK - 1) / kF16BK;

  uint4 areg[D][2][WM][2];  // [ring slot][k-block][32-row tile][slice of the block]
  uint2 breg[D][B_UNITS];
  uint32_t sreg[D][B_UNITS];

  // Per-lane base pointers; everything that changes from stage to stage is a wavefront-uniform
  // offset (scalar registers), so issuing a load costs no vector address arithmetic.
  const int KB = K >> 5;  // 32-k blocks per row
  const uint8_t* a_ptr[WM];
#pragma unroll
  for (int a = 0; a < WM; ++a) {
    int mt = (m0 >> 5) + a;
    const int mt_last = (M - 1) >> 5;
    mt = mt < mt_last ? mt : mt_last;  // tiles past M repeat the last one; never stored
    a_ptr[a] = reinterpret_cast<const uint8_t*>(ah) + (size_t)mt * KB * 2048 + 64 * i32 + 32 * h;
  }
  const uint8_t* bq_ptr[B_UNITS];
  const uint8_t* bs_ptr[B_UNITS];
#pragma unroll
  for (int u = 0; u < B_UNITS; ++u) {
    int nt = nt0 + wave + NWAVES * u;
    nt = nt < NT ? nt : NT - 1;  // tile rows past the matrix: their columns are never stored
    bq_ptr[u] = packed + (size_t)nt * KC * kTileBytes + 16 * lane;
    bs_ptr[u] = hscale + (size_t)nt * KC * kTileScaleBytes + 8 * j;
  }

  // The steady-state loop must stay ONE basic block (the compiler can then wait for exactly
  // the load it needs instead of draining all of them), so nothing below branches: stage
  // numbers and k-blocks are clamped to valid addresses, and what must not contribute is
  // multiplied by a zero scale (padded stages) or meets the zero nibbles and zero scales that
  // pad every weight tile (k >= K).
  auto load_a = [&](int s, uint4 (&dst)[2][WM][2]) {
    const int sc = s < nstages ? s : nstages - 1;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      int blk = 2 * sc + kb;
      blk = blk < KB ? blk : KB - 1;
      const int off = blk * 2048;
#pragma unroll
      for (int a = 0; a < WM; ++a) {
        dst[kb][a][0] = *reinterpret_cast<const uint4*>(a_ptr[a] + off);
        dst[kb][a][1] = *reinterpret_cast<const uint4*>(a_ptr[a] + off + 16);
      }
    }
  };

  auto load_b = [&](int s, uint2 (&q)[B_UNITS], uint32_t (&sc)[B_UNITS]) {
    const int st = s < nstages ? s : nstages - 1;
    const int kc = st >> 1, half = st & 1;
    const int offq = kc * kTileBytes + 8 * half;
    const int offs = kc * kTileScaleBytes + 4 * half;
#pragma unroll
    for (int u = 0; u < B_UNITS; ++u) {
      q[u] = *reinterpret_cast<const uint2*>(bq_ptr[u] + offq);
      sc[u] = *reinterpret_cast<const uint32_t*>(bs_ptr[u] + offs);
    }
  };

  // Tile lane (g, j) of tile row ntl, block dd -> fragment (slice 2*dd + (g & 1), column tile
  // ntl / 2), operand lane 32*(g >> 1) + 16*(ntl & 1) + j.
  // `s` is the stage the registers hold; a stage past the end (loaded from clamped addresses)
  // gets scale 0. The mask is applied here, at use, so that the load itself has no consumer
  // until D stages later.
  auto store_b = [&](int s, int buf, const uint2 (&q)[B_UNITS], const uint32_t (&sc)[B_UNITS]) {
    const uint32_t keep = s < nstages ? 0xFFFFFFFFu : 0u;
    const h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
#pragma unroll
    for (int u = 0; u < B_UNITS; ++u) {
      const int ntl = wave + NWAVES * u;
      const h2 s2 = __builtin_bit_cast(h2, sc[u] & keep);
      const h2 s2_16 = s2 * sixteenth;
      const h2 s_lo = {s2[0], s2[0]}, s_lo16 = {s2_16[0], s2_16[0]};
      const h2 s_hi = {s2[1], s2[1]}, s_hi16 = {s2_16[1], s2_16[1]};
      const int op_lane = 32 * (g >> 1) + 16 * (ntl & 1) + j;
      uint8_t* base = sB + buf * kBufBytes + ((g & 1) * BN32 + (ntl >> 1)) * 1024 + 16 * op_lane;
      *reinterpret_cast<uint4*>(base) = dequant8(q[u].x, s_lo, s_lo16);                    // block 0
      *reinterpret_cast<uint4*>(base + 2 * BN32 * 1024) = dequant8(q[u].y, s_hi, s_hi16);  // block 1
    }
  };

  v16f acc[WM][WN];
#pragma unroll
  for (int a = 0; a < WM; ++a)
#pragma unroll
    for (int b = 0; b < WN; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

  // Prologue: A stages 0..D-1 and B stages 0..D in flight; B stage 0 goes to LDS buffer 0.
#pragma unroll
  for (int p = 0; p < D; ++p) load_a(p, areg[p]);
  {
    uint2 q0[B_UNITS];
    uint32_t s0[B_UNITS];
    load_b(0, q0, s0);
#pragma unroll
    for (int p = 0; p < D; ++p) load_b(p + 1, breg[p], sreg[p]);  // ring slot p holds stage p+1
    store_b(0, 0, q0, s0);
  }

  // Stages are processed D at a time (ring slot u and LDS buffer u & 1 are then compile-time
  // constants); the stage count is rounded up to a multiple of D, extra stages multiply by 0.
  for (int s_base = 0; s_base < nstages; s_base += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int s = s_base + u;
      __syncthreads();
      // B of stage s+1 (ring slot u) -> the LDS buffer not being read; refill the slot
      store_b(s + 1, (u + 1) & 1, breg[u], sreg[u]);
      load_b(s + 1 + D, breg[u], sreg[u]);

      // B fragments come from LDS one k-slice ahead of the MFMAs that use them.
      const uint8_t* bbuf = sB + (u & 1) * kBufBytes + 16 * lane;
      h8 bf[2][WN];
#pragma unroll
      for (int b = 0; b < WN; ++b)
        bf[0][b] = *reinterpret_cast<const h8*>(bbuf + (wn * WN + b) * 1024);
#pragma unroll
      for (int sl = 0; sl < 4; ++sl) {
        if (sl < 3) {
#pragma unroll
          for (int b = 0; b < WN; ++b)
            bf[(sl + 1) & 1][b] =
                *reinterpret_cast<const h8*>(bbuf + ((sl + 1) * BN32 + wn * WN + b) * 1024);
        }
#pragma unroll
        for (int b = 0; b < WN; ++b) {
#pragma unroll
          for (int a = 0; a < WM; ++a) {
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(h8, areg[u][sl >> 1][a][sl & 1]), bf[sl & 1][b], acc[a][b], 0, 0,
                0);
          }
        }
      }
      load_a(s + D, areg[u]);
    }
  }

  // C layout of a 32x32 tile: lane (h, i32) holds column i32; register v holds row
  // 8*(v/4) + 4*h + v%4.
#pragma unroll
  for (int b = 0; b < WN; ++b) {
    const int n = 16 * nt0 + 32 * (wn * WN + b) + i32;
    if (n >= N) continue;
    const float rm = rowmul[n], bs = bias[n];
#pragma unroll
    for (int a = 0; a < WM; ++a) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + 32 * a + 8 * (v >> 2) + 4 * h + (v & 3);
        if (m < M) {
          float val = acc[a][b][v] * rm;
          val = __fmaf_rn(val, recip[m], bs);
          val = fminf(fmaxf(val, -3.402823466e+38f), 3.402823466e+38f);
          y[(size_t)m * N + n] = val;
        }
      }
    }
  }
}

template <int WAVES_M, int WAVES_N, int WM, int WN, int DEPTH>
static hipError_t launch_f16(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                             hipStream_t s) {
  constexpr int BM = 32 * WM * WAVES_M, WNT = 2 * WN * WAVES_N;
  const WeightGeom g = weight_geom(N, K);
  const WsGeom w = ws_geom(M, K);
  const int NB = (g.NT + WNT - 1) / WNT, MB = (M + BM - 1) / BM;
  const int grid = ((MB * NB + 7) / 8) * 8;
  // keep together what is more expensive to fetch eight times: the f16 activations (2 bytes per
  // element) or the packed weights (0.5625 bytes per element)
  const int n_major = (double)M * 2.0 <= (double)N * 0.5625 ? 1 : 0;
  hipLaunchKernelGGL((gemm_f16_kernel<WAVES_M, WAVES_N, WM, WN, DEPTH>), dim3(grid),
                     dim3(64 * WAVES_M * WAVES_N), 0, s, y,
                     reinterpret_cast<const _Float16*>(ws + w.ah_off),
                     reinterpret_cast<const float*>(ws + w.scale_off), packed,
                     packed + g.hscale_off, reinterpret_cast<const float*>(packed + g.rowmul_off),
                     reinterpret_cast<const float*>(packed + g.bias_off), M, N, K, g.NT, g.KC, MB, NB,
                     n_major);
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

// Tile shape by how many 128 x 128 tiles the problem has (measured on MI355X at M = 128..2048 over
// the decoder and ViT shapes). A stage of 64 k costs a workgroup about the same time whatever
// its tile size as long as it is alone on its CU, so few-tile problems take smaller tiles: more
// workgroups, several per CU, which overlap each other's stalls. With many tiles the larger tile's
// operand reuse wins; from 1024 tiles on, 4 wavefronts per workgroup and three workgroups per CU
// did best, below that 8 wavefronts per workgroup.
hipError_t launch_gemm(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                       int kernel, hipStream_t s) {
  if (kernel == kKernelGemmI8 || (kernel == kKernelAuto && M <= 32)) {
    return launch_gemm_i8(y, ws, packed, M, K, N, s);
  }
  const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
  if (tiles < 128) return launch_f16<2, 2, 1, 1, 8>(y, ws, packed, M, K, N, s);   //  64 x  64
  if (tiles < 512) return launch_f16<4, 1, 1, 2, 2>(y, ws, packed, M, K, N, s);   // 128 x  64
  if (tiles < 1024) return launch_f16<4, 2, 1, 2, 2>(y, ws, packed, M, K, N, s);  // 128 x 128, 8 wavefronts
  return launch_f16<4, 1, 1, 4, 2>(y, ws, packed, M, K, N, s);                    // 128 x 128, 4 wavefronts
}

}  // namespace w4
