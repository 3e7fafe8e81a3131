// Prefill product (M > 8): y[M][N] from quantised activation rows and the tiled 4-bit weights.
//
// Two kernels:
//
//  * gemm_f16_kernel (M > 8): v_mfma_f32_32x32x16_f16 on EXACT f16 operands. The activation
//    operand is a_q - zp (an integer in [-255, 255]); the weight operand is q * scale / 2^E_n
//    (4 + 8 significant bits), dequantised ONCE per workgroup from the 4-bit tiles into LDS,
//    already in MFMA fragment order. Every product is exact in f32; only the order of the f32
//    additions differs from the scalar model. No per-block work is left in the MFMA loop, which
//    is what lets the matrix cores run ahead of the VALU: with int8 MFMA every 32-k block would
//    need a convert + scale FMA per accumulator register, and that is VALU-bound.
//
//  * gemm_i8_kernel (selectable by number, a cross-check for the other): integer path. It served
//    9 <= M <= 32 until the f16 kernel's small tiles made that one 2-3 x faster there too.
//
// Integer path: v_mfma_i32_16x16x32_i8. One MFMA spans exactly one scale block (32 k), so the
// block sums are exact int32, as in the reference's scalar model
// (tests/Arm/KaiLinearTest.hpp:342-372); each is converted and scaled in f32 by the block's
// scale. A wavefront owns one 16-row weight tile row and a 64-row slab of activations:
// dword d of its 128-bit weight load is directly the B operand (two mask ops), the A operand
// is 8 consecutive int8 of an activation row.
#include "w4a32_internal.h"

#include <type_traits>

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

#ifndef W4_PAIR_STORE_POLICY
#define W4_PAIR_STORE_POLICY 2
#endif
constexpr int kF16BK = 64;    // k per stage (two scale blocks, half of a weight tile chunk)

typedef float v16f __attribute__((ext_vector_type(16)));

// v_mfma_f32_32x32x16_f16 (8 passes of 4 clocks; measured on MI355X: twice the rate of the
// 16x16x32 shape). Operands: lane l = 32*h + i holds 8 f16 of row/column i at "k-slot" h. Which k
// values a slot stands for is free as long as A and B agree; here, inside a 32-k scale block,
// slice 0 is k {0..7 | 16..23} for h = {0 | 1} and slice 1 is k {8..15 | 24..31}, so that one
// lane's two A operands of a block are 32 contiguous bytes of its activation row.
//
// Workgroup = WAVES_M x WAVES_N wavefronts on a BM x BN tile (BM = 32*WM*WAVES_M,
// BN = 32*WN*WAVES_N); a wavefront owns WM x WN blocks of 32 x 32 outputs.
//
//  * A (f16 activations) never touches LDS: the row quantiser already wrote it as 2 KiB chunks
//    of 32 rows x 32 k, so the two operand loads of a block read one contiguous chunk (instead
//    of 32 rows that lie K*2 bytes apart), into a register ring DEPTH stages deep.
//  * B (4-bit weights) is shared by the wavefronts: its packed bytes are prefetched into a small
//    register ring, dequantised once per workgroup to f16 and double-buffered in LDS as 1 KiB
//    fragments in lane order (lane l at l*16: conflict-free 128-bit accesses).
//  * One barrier per stage: it publishes the B buffer written during the previous stage and
//    frees the one read during it.
//  * What bounds a stage (measured): LDS moves 128 bytes per clock and CU, and a B fragment is
//    read once per WM products, so WM = 1 costs 160 bytes per clock at the full product rate
//    (reads + the tile's own writes): LDS-bound. WM = 2 needs 80. A is read once per WN products
//    through the vector L1 (64 bytes per clock and CU): WN = 4 needs 32.
//
// GROUPED: up to kMaxGemmGroup Linears on the same activation rows in one launch. Their column
// blocks are numbered through (Linear i owns blocks nb_first[i] .. nb_first[i+1]-1); a workgroup
// looks its Linear up and takes N, the blob and the output from the table.
//
// PAIR: two Linears of equal N on the same rows (the MLP's gate and up) whose outputs are only wanted as
// silu(y0) * y1: the left half of a workgroup's column fragments comes from Linear 0, the right half from
// Linear 1, same columns, so that a wavefront holds both factors of an output in the same lane and
// register index; it stores the product (N columns) and neither factor reaches memory.
//
// SPLITK: `ksplit` workgroups share a tile, each takes a contiguous range of the stages and stores
// its raw f32 sums to part[ks][M][N]; splitk_reduce_kernel adds the parts in a fixed order and
// applies the output transform. For problems with few tiles and a long K (down_proj at M <= 512:
// 48 tiles of 128 x 128 for 256 CUs, 140 stages each).
constexpr int kModePlain = 0, kModeGrouped = 1, kModeSplitK = 2, kModePair = 3;
constexpr int kMaxGemmGroup = W4A32_MAX_GROUP;
struct GemmGroup {
  float* y[kMaxGemmGroup];
  const uint8_t* packed[kMaxGemmGroup];
  int N[kMaxGemmGroup];
  int nb_first[kMaxGemmGroup + 1];  // entries past the last Linear hold the total
};

template <int WAVES_M, int WAVES_N, int WM, int WN, int DEPTH, int OCC, int MODE, int BE, int WK>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N * WK, OCC) void gemm_f16_kernel(
    const _Float16* __restrict__ ah, const uint8_t* __restrict__ packed0, const uint8_t* __restrict__ packed1,
    const uint8_t* __restrict__ packed2, int M, int K, int N0, int N1, int N2, unsigned nbs, unsigned nbf,
    unsigned flags,  // 16 dwords: preloaded by the dispatcher
    float* __restrict__ y_arg, const float* __restrict__ recip, float* __restrict__ part, const GemmGroup grp) {
  // Everything a workgroup needs to find its tile and request its first operands arrives in the preloaded
  // registers (a read of the argument segment takes about half a microsecond, in front of every workgroup's
  // first load): the activations, the weights of up to three Linears (plain and split-K: packed0; pair: gate,
  // up) and their widths, from which the tile geometry and the scale / row-factor / bias planes follow, and
  //   nbs   = row blocks | column blocks << 16
  //   nbf   = grouped: first column block of Linear 1 | of Linear 2 << 16
  //   flags = n_major | k-parts << 8 | Linears << 16 | grouped: first column block of Linear 3 << 20
  // Outputs, the activations' row factors, the parts' scratch and a fourth Linear come from the segment and are
  // used in the epilogue.
  const int MB = (int)(nbs & 0xFFFFu), NB = (int)(nbs >> 16);
  const int n_major = (int)(flags & 1u), ksplit = (int)((flags >> 8) & 0xFFu);
  const int KC = (K + kTileK - 1) / kTileK;
  constexpr bool GROUPED = MODE == kModeGrouped, SPLITK = MODE == kModeSplitK, PAIR = MODE == kModePair;
  static_assert(!PAIR || (WAVES_N == 1 && WN % 2 == 0 && WK == 1), "a wavefront must own both halves");
  constexpr int D = DEPTH;
  // BE = stages per barrier (1 or 2). The loop is unrolled U stages at a time so that ring slots and
  // LDS buffers are compile-time constants.
  static_assert(BE == 1 || (BE == 2 && D == 2), "two stages per barrier are built for a ring of two");
  constexpr int U = BE == 2 ? 4 : (D < 2 ? 2 : D);
  static_assert(U % (2 * BE) == 0, "the unrolled stages must cover whole pairs of LDS buffer sets");
  static_assert(WK == 1 || WK == 2, "one or two sets of wavefronts per stage");
  constexpr int NWAVES = WAVES_M * WAVES_N * WK;
  constexpr int BM = 32 * WM * WAVES_M;
  constexpr int BN32 = WN * WAVES_N;           // 32-column fragments per workgroup and k-slice
  constexpr int WNT = 2 * BN32;                // 16-row weight tile rows per workgroup
  // Wavefront w dequantises tile rows w, w + NWAVES, ... of the stage. When that does not come out even,
  // the surplus units repeat a valid row's loads and write to a spare fragment nobody reads.
  constexpr int B_UNITS = (WNT + NWAVES - 1) / NWAVES;  // 8-byte pieces of packed B per thread per stage
  constexpr bool kSpareUnits = WNT % NWAVES != 0;
  constexpr int kBufBytes = 4 * BN32 * 1024;   // one B stage: [4 k-slices][BN32 fragments]
  constexpr int SL = 4 / WK;                   // k-slices of a stage that one wavefront multiplies
  constexpr int AKB = 2 / WK;                  // activation k-blocks (32 k) of a stage, likewise
  constexpr int kMfma = SL * WM * WN;          // products per wavefront and stage
  constexpr int NDW = 2 * B_UNITS;             // packed dwords a thread dequantises per stage
  constexpr int NSTEP = 4 * NDW;               // in four steps each
  constexpr int kLdsBufs = 2 * BE;             // two sets (read / being written) of BE stage buffers
  constexpr int kSpareOff = kLdsBufs * kBufBytes;
  constexpr int kStageBytes = kSpareOff + (kSpareUnits ? 1024 : 0);
  constexpr int kMeetBytes = WK == 2 ? NWAVES * 4096 : 0;  // the k-halves' sums meet in the same memory
  constexpr int kLdsBytes = kStageBytes > kMeetBytes ? kStageBytes : kMeetBytes;
  static_assert(kLdsBytes <= 65536, "static LDS");

  __shared__ __align__(16) uint8_t sB[kLdsBytes];

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // scalar: what derives from it is too
  // WK = 2: wavefronts wave and wave + NWAVES/2 own the same outputs and each take one 32-k block of
  // every stage (two wavefronts per SIMD when the workgroup has a CU to itself; their sums meet in LDS
  // after the loop).
  const int wk = wave / (WAVES_M * WAVES_N);
  const int wm = (wave % (WAVES_M * WAVES_N)) / WAVES_N, wn = wave % WAVES_N;
  const int g = lane >> 4, j = lane & 15;     // position inside a weight tile
  const int h = lane >> 5, i32 = lane & 31;   // position inside an MFMA operand / C tile
  // Workgroup -> tile. The hardware deals consecutive workgroups round-robin to the 8 XCDs, each
  // with its own L2. Workgroup b therefore takes tile (b % 8) * ceil(T / 8) + b / 8, so that an
  // XCD owns one contiguous run of tiles; the run is ordered so that neighbours share the larger
  // operand (n_major: all row blocks of a weight column block together, weights fetched by one
  // XCD only; otherwise all column blocks of a row block together).
  const int total = MB * NB * (SPLITK ? ksplit : 1);
  const int per_xcd = (total + 7) >> 3;
  int tile = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
  if (tile >= total) return;  // whole workgroup: no barrier has been reached yet
  int ks = 0;
  if constexpr (SPLITK) {
    ks = tile % ksplit;
    tile /= ksplit;
  }
  const int mb = n_major ? tile % MB : tile / NB;
  int nb = n_major ? tile / MB : tile % NB;
  float* y = y_arg;
  const uint8_t* packed = packed0;
  int N = N0;
  if constexpr (GROUPED) {
    const int count = (int)((flags >> 16) & 0xFu);
    const int f1 = (int)(nbf & 0xFFFFu), f2 = (int)(nbf >> 16), f3 = (int)(flags >> 20);
    y = grp.y[0];
    if (count > 1 && nb >= f1) {
      packed = packed1;
      N = N1;
      y = grp.y[1];
    }
    if (count > 2 && nb >= f2) {
      packed = packed2;
      N = N2;
      y = grp.y[2];
    }
    if (count > 3 && nb >= f3) {
      packed = grp.packed[3];
      N = grp.N[3];
      y = grp.y[3];
    }
    nb -= count > 3 && nb >= f3 ? f3 : count > 2 && nb >= f2 ? f2 : count > 1 && nb >= f1 ? f1 : 0;
  }
  const WeightGeom wgm = weight_geom(N, K);
  const int NT = wgm.NT;
  const uint8_t* hscale = packed + wgm.hscale_off;
  const float* rowmul = reinterpret_cast<const float*>(packed + wgm.rowmul_off);
  const float* bias = reinterpret_cast<const float*>(packed + wgm.bias_off);
  const int m0 = mb * BM + 32 * WM * wm;
  // first 16-row weight tile row of this workgroup's columns (PAIR: in both Linears, half the units each)
  const int nt0 = nb * (PAIR ? WNT / 2 : WNT);
  // this workgroup's stages: [s_begin, nstages)
  int s_begin = 0, nstages = (K + kF16BK - 1) / kF16BK;
  if constexpr (SPLITK) {
    // whole pairs of stages (one 128-k weight chunk): a range starts on an even stage, which makes the
    // half of the chunk that a stage of the unrolled loop reads a compile-time constant
    const int npairs = (nstages + 1) >> 1;
    const int s_end = 2 * (int)((long)(ks + 1) * npairs / ksplit);
    s_begin = 2 * (int)((long)ks * npairs / ksplit);
    nstages = s_end < nstages ? s_end : nstages;
  }

  uint4 areg[D][AKB][WM][2];  // [ring slot][k-block][32-row tile][slice of the block]
  uint2 breg[D][B_UNITS];
  uint32_t sreg[D][B_UNITS];

  // Per-lane pointers. In the steady-state loop they advance by constants and a stage's loads use
  // immediate offsets; elsewhere what changes from stage to stage is a wavefront-uniform offset.
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
    int ntl = wave + NWAVES * u;
    ntl = ntl < WNT ? ntl : WNT - 1;  // a surplus unit
    const uint8_t* pk = packed;
    const uint8_t* hs = hscale;
    if constexpr (PAIR) {
      const int side = ntl >= WNT / 2 ? 1 : 0;  // wavefront-uniform
      ntl -= side * (WNT / 2);
      pk = side ? packed1 : packed0;
      hs = pk + wgm.hscale_off;
    }
    int nt = nt0 + ntl;
    nt = nt < NT ? nt : NT - 1;  // tile rows past the matrix: their columns are never stored
    bq_ptr[u] = pk + (size_t)nt * KC * kTileBytes + 16 * lane;
    bs_ptr[u] = hs + (size_t)nt * KC * kTileScaleBytes + 8 * j;
  }

  // The loops must stay ONE basic block each (the compiler can then wait for exactly the load it
  // needs instead of draining all of them), so nothing below branches. The steady-state loop runs
  // while every stage it loads exists: its pointers advance by constants and no address is computed.
  // The prologue and the last iterations load through the clamped forms below: stage numbers and
  // k-blocks are clamped to valid addresses, and what must not contribute is multiplied by a zero
  // scale (padded stages) or meets the zero nibbles and zero scales that pad every weight tile
  // (k >= K). a_pos, bq_pos and bs_pos are the bytes by which the per-lane pointers have advanced.
  int a_pos = 0, bq_pos = 0, bs_pos = 0;
  auto load_a_kb = [&](int s, int kbl, uint4 (&dst)[AKB][WM][2]) {
    const int sc = s < nstages ? s : nstages - 1;
    int blk = 2 * sc + (WK == 2 ? wk : kbl);
    blk = blk < KB ? blk : KB - 1;
    const int off = blk * 2048 - a_pos;
#pragma unroll
    for (int a = 0; a < WM; ++a) {
      dst[kbl][a][0] = *reinterpret_cast<const uint4*>(a_ptr[a] + off);
      dst[kbl][a][1] = *reinterpret_cast<const uint4*>(a_ptr[a] + off + 16);
    }
  };
  // steady state: a_ptr stands at k-block 2 * (the stage to load) (+ wk)
  auto load_a_kb_next = [&](int kbl, uint4 (&dst)[AKB][WM][2]) {
#pragma unroll
    for (int a = 0; a < WM; ++a) {
      dst[kbl][a][0] = *reinterpret_cast<const uint4*>(a_ptr[a] + kbl * 2048);
      dst[kbl][a][1] = *reinterpret_cast<const uint4*>(a_ptr[a] + kbl * 2048 + 16);
    }
  };

  auto load_b = [&](int s, uint2 (&q)[B_UNITS], uint32_t (&sc)[B_UNITS]) {
    const int st = s < nstages ? s : nstages - 1;
    const int kc = st >> 1, half = st & 1;
    const int offq = kc * kTileBytes + 8 * half - bq_pos;
    const int offs = kc * kTileScaleBytes + 4 * half - bs_pos;
#pragma unroll
    for (int u = 0; u < B_UNITS; ++u) {
      const u32x2 t2 = load_global<u32x2>(bq_ptr[u] + offq);  // (a table pointer is a generic one)
      q[u] = make_uint2(t2.x, t2.y);
      sc[u] = load_global<uint32_t>(bs_ptr[u] + offs);
    }
  };
  // steady state: the pointers stand at the chunk of the iteration's first stage, `rel` (a constant
  // after unrolling) is the stage to load counted from there
  auto load_b_rel = [&](int rel, uint2 (&q)[B_UNITS], uint32_t (&sc)[B_UNITS]) {
    const int offq = (rel >> 1) * kTileBytes + 8 * (rel & 1);
    const int offs = (rel >> 1) * kTileScaleBytes + 4 * (rel & 1);
#pragma unroll
    for (int u = 0; u < B_UNITS; ++u) {
      const u32x2 t2 = load_global<u32x2>(bq_ptr[u] + offq);
      q[u] = make_uint2(t2.x, t2.y);
      sc[u] = load_global<uint32_t>(bs_ptr[u] + offs);
    }
  };

  // Tile lane (g, j) of tile row ntl, block dd -> fragment (slice 2*dd + (g & 1), column tile
  // ntl / 2), operand lane 32*(g >> 1) + 16*(ntl & 1) + j.
  auto frag_ptr = [&](int buf, int unit, int dd) {
    const int ntl = wave + NWAVES * unit;
    const int op_lane = 32 * (g >> 1) + 16 * (ntl & 1) + j;
    const int off = buf * kBufBytes + ((2 * dd + (g & 1)) * BN32 + (ntl >> 1)) * 1024;
    return sB + (kSpareUnits && ntl >= WNT ? kSpareOff : off) + 16 * op_lane;
  };

  v16f acc[WM][WN];
#pragma unroll
  for (int a = 0; a < WM; ++a)
#pragma unroll
    for (int b = 0; b < WN; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

  // Prologue: the first D stages of A and D+1 of B in flight; the first B stage goes to LDS buffer 0. The
  // loads are issued in the loop's own order (per stage: B, then A): the compiler derives each
  // wait in the loop from the fewest loads that can be younger than the one it needs on any way
  // into the loop, so a prologue with another order makes the loop wait for newer loads than it
  // uses.
  // B runs BE stages ahead of the products: the first BE stages go to the first buffer set here, and
  // ring slot p holds stage p + BE.
  {
    uint2 q0[BE][B_UNITS];
    uint32_t s0[BE][B_UNITS];
#pragma unroll
    for (int e = 0; e < BE; ++e) load_b(s_begin + e, q0[e], s0[e]);
#pragma unroll
    for (int p = 0; p < D; ++p) {
      load_b(s_begin + p + BE, breg[p], sreg[p]);
#pragma unroll
      for (int kbl = 0; kbl < AKB; ++kbl) load_a_kb(s_begin + p, kbl, areg[p]);
    }
    __builtin_amdgcn_sched_barrier(0);
    const h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
#pragma unroll
    for (int e = 0; e < BE; ++e) {
      const uint32_t keep = s_begin + e < nstages ? 0xFFFFFFFFu : 0u;
#pragma unroll
      for (int u = 0; u < B_UNITS; ++u) {
        const h2 s2 = __builtin_bit_cast(h2, s0[e][u] & keep);
        const h2 s2_16 = s2 * sixteenth;
        *reinterpret_cast<uint4*>(frag_ptr(e, u, 0)) =
            dequant8(q0[e][u].x, h2{s2[0], s2[0]}, h2{s2_16[0], s2_16[0]});
        *reinterpret_cast<uint4*>(frag_ptr(e, u, 1)) =
            dequant8(q0[e][u].y, h2{s2[1], s2[1]}, h2{s2_16[1], s2_16[1]});
      }
    }
  }

  // Stages are processed D at a time (ring slot u and LDS buffer u & 1 are then compile-time
  // constants); the stage count is rounded up to a multiple of D, extra stages multiply by 0.
  //
  // The order inside a stage is written out and fenced (sched_barrier) product by product: a
  // product occupies the matrix pipe for 32 clocks but its issue slot for 4, so the same
  // wavefront dequantises the next stage's weights, a few instructions at a time, and issues its
  // LDS and global traffic in the gaps between its own products. (Left to the scheduler, all of a
  // stage's dequantisation ran first and the products after it.)
  //
  // With BE = 2 the barrier comes every second stage (four LDS buffers): the stage behind it finds its
  // first fragments requested under the previous stage's last products, and a lone workgroup on a CU
  // pays the barrier and that LDS round trip half as often.
  //
  // Dequantisation of a packed dword (eight two's complement nibbles n): (dword & 0x000F000F) ^ 0x64086408
  // is the f16 pair 1024 + (n ^ 8) of nibbles 0 and 4 in one three-input bit operation, likewise
  // 0x00F000F0 / 0x64806480 for 1024 + 16 (n ^ 8) of nibbles 1 and 5, and the same on the dword >> 8;
  // minus 1032 (1152) that is n exactly, times the scale (scale / 16) the weight: 13 instructions for
  // eight weights. The two constants sit in vector registers (an instruction reads one scalar operand).
  uint32_t k_lo = 0x64086408u, k_hi = 0x64806480u;
  asm volatile("" : "+v"(k_lo), "+v"(k_hi));
  h8 bf[2][WN];
  // Three forms of U stages. kSteady: every load is in range and goes through the advancing pointers.
  // kClamped: any stage may lie past the end. kLast: the U stages are exactly the last ones, so what lies
  // past the end is known at compile time and neither loaded nor dequantised.
  constexpr int kSteady = 0, kClamped = 1, kLast = 2;
  auto run_stages = [&](auto form_tag, const int s_base) __attribute__((always_inline)) {
    constexpr int FORM = decltype(form_tag)::value;
    constexpr bool TAIL = FORM != kSteady;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = s_base + u;
      constexpr int kSlotMask = D - 1;
      static_assert((D & (D - 1)) == 0, "ring slot = stage mod D by masking");
      const int slot = u & kSlotMask;
      const int rbuf = ((u / BE) & 1) * BE + u % BE;                    // buffer this stage reads
      const int wbuf = (((u + BE) / BE) & 1) * BE + (u + BE) % BE;      // buffer of stage s + BE
      const uint8_t* bbuf = sB + rbuf * kBufBytes + 16 * lane + (WK == 2 ? wk * (SL * BN32 * 1024) : 0);
      // B fragments are requested LA products before their use, one per product (a steady stream of LDS
      // reads; measured the same for LA = 1..4, and the same as a whole slice at a time). A fragment's
      // register is that of the fragment two slices before it, which must have been used: LA <= 2 WN.
      constexpr int F = SL * WN;  // fragments of a stage; fragment f = slice f / WN, column block f % WN
      constexpr int LA = 2;
      static_assert(LA <= 2 * WN && LA < F, "a fragment would overwrite one that is still to be used");
      auto fetch = [&](int f, const uint8_t* base) {
        bf[(f / WN) & 1][f % WN] =
            *reinterpret_cast<const h8*>(base + ((f / WN) * BN32 + wn * WN + f % WN) * 1024);
      };
      if (u % BE == 0) {
        __syncthreads();
#pragma unroll
        for (int f = 0; f < LA; ++f) fetch(f, bbuf);
        __builtin_amdgcn_sched_barrier(0);  // requested first: their latency covers what follows
      }
      // Inputs of the dequantisation (stage s + BE, in this stage's ring slot); the slot then takes its
      // next load. A stage past the end (loaded from clamped addresses) gets scale 0.
      uint32_t dx[NDW];
      h2 dsc[NDW], dsc16[NDW];
      {
        const uint32_t keep = FORM != kClamped || s + BE < nstages ? 0xFFFFFFFFu : 0u;
        const h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
#pragma unroll
        for (int q = 0; q < B_UNITS; ++q) {
          const h2 s2 = __builtin_bit_cast(h2, FORM == kClamped ? sreg[slot][q] & keep : sreg[slot][q]);
          const h2 s2_16 = s2 * sixteenth;
          dsc[2 * q] = h2{s2[0], s2[0]};
          dsc16[2 * q] = h2{s2_16[0], s2_16[0]};
          dsc[2 * q + 1] = h2{s2[1], s2[1]};
          dsc16[2 * q + 1] = h2{s2_16[1], s2_16[1]};
          dx[2 * q] = breg[slot][q].x;
          dx[2 * q + 1] = breg[slot][q].y;
        }
      }
      const bool dequantise = FORM != kLast || u + BE < U;  // (after unrolling: a constant)
      if constexpr (FORM == kSteady) {
        load_b_rel(u + BE + D, breg[slot], sreg[slot]);
      } else {
        if (FORM != kLast || u + BE + D < U) load_b(s + BE + D, breg[slot], sreg[slot]);
      }
      __builtin_amdgcn_sched_barrier(0);
      // Four steps per dword d (unit d / 2, scale block d % 2). A step never multiplies what it has just
      // subtracted: a product that reads half of a register the instruction before it wrote costs a
      // wait state.
      h2 dlo[NDW], dhi[NDW];
      uint32_t dxh[NDW];
      uint4 dout[NDW];
      auto dq_step = [&](int idx) {
        const int d = idx >> 2, ph = idx & 3;
        const h2 b1 = {(_Float16)1032.0f, (_Float16)1032.0f};
        const h2 b16 = {(_Float16)1152.0f, (_Float16)1152.0f};
        if (ph == 0) {
          dlo[d] = __builtin_bit_cast(h2, (dx[d] & 0x000F000Fu) ^ k_lo) - b1;
          dhi[d] = __builtin_bit_cast(h2, (dx[d] & 0x00F000F0u) ^ k_hi) - b16;
        } else if (ph == 1) {
          dout[d].x = __builtin_bit_cast(uint32_t, dlo[d] * dsc[d]);
          dout[d].y = __builtin_bit_cast(uint32_t, dhi[d] * dsc16[d]);
          dxh[d] = dx[d] >> 8;
        } else if (ph == 2) {
          dlo[d] = __builtin_bit_cast(h2, (dxh[d] & 0x000F000Fu) ^ k_lo) - b1;
          dhi[d] = __builtin_bit_cast(h2, (dxh[d] & 0x00F000F0u) ^ k_hi) - b16;
        } else {
          dout[d].z = __builtin_bit_cast(uint32_t, dlo[d] * dsc[d]);
          dout[d].w = __builtin_bit_cast(uint32_t, dhi[d] * dsc16[d]);
          *reinterpret_cast<uint4*>(frag_ptr(wbuf, d >> 1, d & 1)) = dout[d];
        }
      };
      int mi = 0;
#pragma unroll
      for (int sl = 0; sl < SL; ++sl) {
#pragma unroll
        for (int b = 0; b < WN; ++b) {
#pragma unroll
          for (int a = 0; a < WM; ++a) {
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(h8, areg[slot][sl >> 1][a][sl & 1]), bf[sl & 1][b], acc[a][b], 0, 0, 0);
            if (a == 0) {
              const int f = sl * WN + b + LA;
              if (f < F) {
                fetch(f, bbuf);
              } else if ((u + 1) % BE != 0) {  // no barrier ahead: the next stage's first fragments
                fetch(f - F, bbuf + kBufBytes);
              }
            }
#pragma unroll
            for (int st = mi * NSTEP / kMfma; st < (mi + 1) * NSTEP / kMfma; ++st) {
              if (dequantise) dq_step(st);
            }
            ++mi;
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if (sl & 1) {  // that k-block's registers are free now
          if constexpr (TAIL) {
            if (FORM != kLast || u + D < U) load_a_kb(s + D, sl >> 1, areg[slot]);
          } else {
            load_a_kb_next(sl >> 1, areg[slot]);
          }
        }
      }
      if constexpr (FORM == kSteady) {
#pragma unroll
        for (int a = 0; a < WM; ++a) a_ptr[a] += 4096;
      }
    }
    if constexpr (FORM == kSteady) {
#pragma unroll
      for (int q = 0; q < B_UNITS; ++q) {
        bq_ptr[q] += (U / 2) * kTileBytes;
        bs_ptr[q] += (U / 2) * kTileScaleBytes;
      }
    }
  };

  int s_base = s_begin;
  if (s_base + U + BE + D <= nstages) {
    // a_ptr to the first stage the loop loads, the weight pointers to the chunk of its first stage
    // (s_begin is even, and so is U: stage s_base + u lies u stages into that chunk)
#pragma unroll
    for (int a = 0; a < WM; ++a) a_ptr[a] += (size_t)(s_begin + D) * 4096 + (WK == 2 ? wk * 2048 : 0);
#pragma unroll
    for (int q = 0; q < B_UNITS; ++q) {
      bq_ptr[q] += (size_t)(s_begin >> 1) * kTileBytes;
      bs_ptr[q] += (size_t)(s_begin >> 1) * kTileScaleBytes;
    }
    // the last stage loaded is s_base + U - 1 + BE + D; BE >= 1 also keeps the activations' last
    // k-block (absent when K / 32 is odd) out of this loop
    for (; s_base + U + BE + D <= nstages; s_base += U) {
      run_stages(std::integral_constant<int, kSteady>{}, s_base);
    }
    a_pos = (s_base + D) * 4096 + (WK == 2 ? wk * 2048 : 0);
    bq_pos = (s_base >> 1) * kTileBytes;
    bs_pos = (s_base >> 1) * kTileScaleBytes;
  }
  // the stages come in whole iterations (a range without stages runs nothing)
  const bool whole = nstages > s_begin && (nstages - s_begin) % U == 0;
  for (; s_base + (whole ? U : 0) < nstages; s_base += U) {
    run_stages(std::integral_constant<int, kClamped>{}, s_base);
  }
  if (whole) run_stages(std::integral_constant<int, kLast>{}, s_base);

  // WK = 2: the two k-halves of an output block meet in LDS, one 32 x 32 block per wavefront and round
  // (4 KiB each, in the stage buffers). The first half keeps column blocks 0..BH-1 and hands over the
  // rest, the second half the other way round; every sum is (first half) + (second half).
  constexpr int BH = WK == 2 ? (WN + 1) / 2 : WN;
  if constexpr (WK == 2) {
    float* xmine = reinterpret_cast<float*>(sB) + wave * 1024 + 4 * lane;
    const float* xpeer = reinterpret_cast<const float*>(sB) + (wave ^ (NWAVES / 2)) * 1024 + 4 * lane;
#pragma unroll
    for (int ra = 0; ra < BH * WM; ++ra) {
      const int r = ra / WM, a = ra % WM;
      const int give0 = BH + r < WN ? BH + r : WN - 1;  // block the first half hands over in this round
      __syncthreads();  // the loop's (then the previous round's) reads of these bytes are over
      if (wk == 0) {
        if (BH + r < WN) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *reinterpret_cast<float4*>(xmine + 256 * q) = make_float4(
                acc[a][give0][4 * q], acc[a][give0][4 * q + 1], acc[a][give0][4 * q + 2], acc[a][give0][4 * q + 3]);
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<float4*>(xmine + 256 * q) =
              make_float4(acc[a][r][4 * q], acc[a][r][4 * q + 1], acc[a][r][4 * q + 2], acc[a][r][4 * q + 3]);
      }
      __syncthreads();
      if (wk == 0) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 o = *reinterpret_cast<const float4*>(xpeer + 256 * q);
          acc[a][r][4 * q] += o.x; acc[a][r][4 * q + 1] += o.y;
          acc[a][r][4 * q + 2] += o.z; acc[a][r][4 * q + 3] += o.w;
        }
      } else if (BH + r < WN) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 o = *reinterpret_cast<const float4*>(xpeer + 256 * q);
          acc[a][give0][4 * q] = o.x + acc[a][give0][4 * q];
          acc[a][give0][4 * q + 1] = o.y + acc[a][give0][4 * q + 1];
          acc[a][give0][4 * q + 2] = o.z + acc[a][give0][4 * q + 2];
          acc[a][give0][4 * q + 3] = o.w + acc[a][give0][4 * q + 3];
        }
      }
    }
  }

  // Everything the output transform reads is loaded before the first store: loads and stores
  // retire through one in-order counter, so a load issued after a store would wait for that store
  // to reach memory.
  float rc[WM][16], rm[WN], bs[WN];
  constexpr int WNH = PAIR ? WN / 2 : WN;  // column blocks a wavefront stores
#pragma unroll
  for (int a = 0; a < WM; ++a) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + 32 * a + 8 * (v >> 2) + 4 * h + (v & 3);
      rc[a][v] = recip[m < M ? m : M - 1];
    }
  }
#pragma unroll
  for (int b = 0; b < WN; ++b) {
    const int n = 16 * nt0 + 32 * (wn * WN + b % WNH) + i32;
    const float* rmp = rowmul;
    const float* bsp = bias;
    if constexpr (PAIR) {
      const uint8_t* pk = b / WNH ? packed1 : packed0;
      rmp = reinterpret_cast<const float*>(pk + wgm.rowmul_off);
      bsp = reinterpret_cast<const float*>(pk + wgm.bias_off);
    }
    rm[b] = load_global<float>(rmp + (n < N ? n : N - 1));
    bs[b] = load_global<float>(bsp + (n < N ? n : N - 1));
  }

  // SPLITK without an output (y == nullptr): the parts are stored with the row and column factors applied
  // (the reader adds them up and adds the bias); with an output they are raw sums (factors 1).
  const bool scaled_parts = SPLITK && y_arg == nullptr;
  float part_rm[WN];
#pragma unroll
  for (int b = 0; b < WN; ++b) part_rm[b] = scaled_parts ? rm[b] : 1.0f;

  __builtin_amdgcn_sched_barrier(0);

  // C layout of a 32x32 tile: lane (h, i32) holds column i32; register v holds row
  // 8*(v/4) + 4*h + v%4. Stores go through a buffer descriptor that covers exactly this
  // workgroup's valid rows: the hardware drops a store whose offset lies past the descriptor's
  // size, so rows >= M need no branch (columns >= N get an offset past the end instead).
  // Straight-line stores matter: with a branch around each one the compiler cannot count
  // outstanding stores and waits for all of them before every use of a loaded factor (that made
  // the epilogue of a 128 x 128 tile take 9 us instead of 1.7).
  // The outputs of a whole Linear are stored non-temporally (cache policy bit 1): they are many times the L2's
  // size and all tiles store at the same moment (gate_proj: M = 512 23.0 -> 21.0 us, M = 1024 38.1 -> 36.4 us, no
  // change from M = 2048 on); split-K parts, which the next kernel reads back at once, stay cached.
  constexpr int kStorePolicy = SPLITK ? 0 : (PAIR ? W4_PAIR_STORE_POLICY : 2);
  const int wg_m0 = mb * BM;
  const int rows_valid = (M - wg_m0 < BM ? M - wg_m0 : BM);
  float* out_base = SPLITK ? part + ((size_t)ks * M + wg_m0) * N : y + (size_t)wg_m0 * N;
  const __amdgpu_buffer_rsrc_t out_rows = __builtin_amdgcn_make_buffer_rsrc(
      out_base, 0, (int)((unsigned)rows_valid * (unsigned)N * 4u), 0x00020000);
  const unsigned row_bytes = (unsigned)N * 4u;
#pragma unroll
  for (int b = 0; b < WNH; ++b) {
    constexpr int kPastEnd = 0x7FFFFFF0;
    const int n = 16 * nt0 + 32 * (wn * WN + b) + i32;
    if (WK == 2 && (b < BH) != (wk == 0)) continue;  // the other k-half stores this block
#pragma unroll
    for (int a = 0; a < WM; ++a) {
      const unsigned row0 = (unsigned)(32 * WM * wm + 32 * a + 4 * h);
      const unsigned off0 = row0 * row_bytes + (unsigned)n * 4u;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float val = acc[a][b][v];
        if constexpr (!SPLITK) {
          val = __fmaf_rn(val * rm[b], rc[a][v], bs[b]);
          val = fminf(fmaxf(val, -3.402823466e+38f), 3.402823466e+38f);
        } else {
          val = val * part_rm[b] * (scaled_parts ? rc[a][v] : 1.0f);
        }
        if constexpr (PAIR) {
          float up = __fmaf_rn(acc[a][b + WNH][v] * rm[b + WNH], rc[a][v], bs[b + WNH]);
          up = fminf(fmaxf(up, -3.402823466e+38f), 3.402823466e+38f);
          val = silu_mul(val, up);
        }
        const unsigned dm = 8 * (v >> 2) + (v & 3);  // row offset from row0
        const int off = n < N ? (int)(off0 + dm * row_bytes) : kPastEnd;
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), out_rows, off, 0, kStorePolicy);
      }
    }
  }
}

// y[m][n] = transform(part[0][m][n] + part[1][m][n] + ...), four columns per thread when N allows.
template <int VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(
    float* __restrict__ y, const float* __restrict__ part, int ksplit, int M, int N,
    const float* __restrict__ recip, const float* __restrict__ rowmul, const float* __restrict__ bias) {
  const size_t total = (size_t)M * N;
  const size_t e = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (e >= total) return;
  const int m = (int)(e / N), n = (int)(e % N);
  float sum[VEC];
  if constexpr (VEC == 4) {
    const float4 p = *reinterpret_cast<const float4*>(part + e);
    sum[0] = p.x; sum[1] = p.y; sum[2] = p.z; sum[3] = p.w;
    for (int k = 1; k < ksplit; ++k) {
      const float4 q = *reinterpret_cast<const float4*>(part + (size_t)k * total + e);
      sum[0] += q.x; sum[1] += q.y; sum[2] += q.z; sum[3] += q.w;
    }
  } else {
    sum[0] = part[e];
    for (int k = 1; k < ksplit; ++k) sum[0] += part[(size_t)k * total + e];
  }
  const float rc = recip[m];
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    float val = __fmaf_rn(sum[i] * rowmul[n + i], rc, bias[n + i]);
    sum[i] = fminf(fmaxf(val, -3.402823466e+38f), 3.402823466e+38f);
  }
  if constexpr (VEC == 4) {
    *reinterpret_cast<float4*>(y + e) = make_float4(sum[0], sum[1], sum[2], sum[3]);
  } else {
    y[e] = sum[0];
  }
}

// One Linear (group == nullptr) or the Linears of `group`, whose column blocks add up to nb_total.
// ksplit > 1: the stages of every tile are dealt to ksplit workgroups (partial sums in `part`).
template <int WAVES_M, int WAVES_N, int WM, int WN, int DEPTH, int OCC, int BE = 1, int WK = 1>
static hipError_t launch_f16(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                             const GemmGroup* group, const int* group_N, int count, int ksplit,
                             float* part, hipStream_t s) {
  constexpr int BM = 32 * WM * WAVES_M, WNT = 2 * WN * WAVES_N;
  const WsGeom w = ws_geom(M, K);
  const int MB = (M + BM - 1) / BM;
  const _Float16* ah = reinterpret_cast<const _Float16*>(ws + w.ah_off);
  const float* recip = reinterpret_cast<const float*>(ws + w.scale_off);
  if (group) {
    GemmGroup g = *group;
    int nb = 0;
    long n_total = 0;
    for (int i = 0; i <= kMaxGemmGroup; ++i) {
      g.nb_first[i] = nb;
      if (i < count) {
        nb += (weight_geom(group_N[i], K).NT + WNT - 1) / WNT;
        n_total += group_N[i];
      }
    }
    const int NB = nb;
    const int n_major = (double)M * 2.0 <= (double)n_total * 0.5625 ? 1 : 0;
    const int f3 = count > 3 ? g.nb_first[3] : 0;  // the boundary in front of a fourth Linear has 12 bits
    if (MB > 0xFFFF || NB > 0xFFFF || f3 > 0xFFF) return hipErrorInvalidValue;
    const unsigned nbs = (unsigned)MB | (unsigned)NB << 16;
    const unsigned nbf = (unsigned)g.nb_first[1] | (unsigned)g.nb_first[2] << 16;
    const unsigned flags = (unsigned)n_major | 1u << 8 | (unsigned)count << 16 | (unsigned)f3 << 20;
    hipLaunchKernelGGL((gemm_f16_kernel<WAVES_M, WAVES_N, WM, WN, DEPTH, OCC, kModeGrouped, BE, WK>),
                       dim3(((MB * NB + 7) / 8) * 8), dim3(64 * WAVES_M * WAVES_N * WK), 0, s, ah, g.packed[0],
                       g.packed[1], g.packed[2], M, K, group_N[0], count > 1 ? group_N[1] : 0,
                       count > 2 ? group_N[2] : 0, nbs, nbf, flags, nullptr, recip, nullptr, g);
    return hipGetLastError();
  }
  const WeightGeom g = weight_geom(N, K);
  const int NB = (g.NT + WNT - 1) / WNT;
  // keep together what is more expensive to fetch eight times: the f16 activations (2 bytes per
  // element) or the packed weights (0.5625 bytes per element)
  const int n_major = (double)M * 2.0 <= (double)N * 0.5625 ? 1 : 0;
  const float* rowmul = reinterpret_cast<const float*>(packed + g.rowmul_off);
  const float* bias = reinterpret_cast<const float*>(packed + g.bias_off);
  if (MB > 0xFFFF || NB > 0xFFFF || ksplit > 0xFF) return hipErrorInvalidValue;
  const unsigned nbs = (unsigned)MB | (unsigned)NB << 16;
  const unsigned flags = (unsigned)n_major | (unsigned)(ksplit > 1 ? ksplit : 1) << 8 | 1u << 16;
  if (ksplit > 1) {
    hipLaunchKernelGGL((gemm_f16_kernel<WAVES_M, WAVES_N, WM, WN, DEPTH, OCC, kModeSplitK, BE, WK>),
                       dim3(((MB * NB * ksplit + 7) / 8) * 8), dim3(64 * WAVES_M * WAVES_N * WK), 0, s, ah,
                       packed, nullptr, nullptr, M, K, N, 0, 0, nbs, 0u, flags, y, recip, part, GemmGroup{});
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    if (!y) return hipSuccess;  // the caller's next kernel adds the (scaled) parts up
    const size_t total = (size_t)M * N;
    if (N % 4 == 0) {
      hipLaunchKernelGGL(splitk_reduce_kernel<4>, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256),
                         0, s, y, part, ksplit, M, N, recip, rowmul, bias);
    } else {
      hipLaunchKernelGGL(splitk_reduce_kernel<1>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                         s, y, part, ksplit, M, N, recip, rowmul, bias);
    }
    return hipGetLastError();
  }
  hipLaunchKernelGGL((gemm_f16_kernel<WAVES_M, WAVES_N, WM, WN, DEPTH, OCC, kModePlain, BE, WK>),
                     dim3(((MB * NB + 7) / 8) * 8), dim3(64 * WAVES_M * WAVES_N * WK), 0, s, ah, packed, nullptr,
                     nullptr, M, K, N, 0, 0, nbs, 0u, flags, y, recip, nullptr, GemmGroup{});
  return hipGetLastError();
}

// silu(x W0^T) * (x W1^T) for two Linears of equal N, stored to one [M][N] output.
template <int WAVES_M, int WN, int DEPTH, int OCC, int WM = 1>
static hipError_t launch_f16_pair(float* act, const uint8_t* ws, const uint8_t* gate, const uint8_t* up, int M,
                                  int K, int N, hipStream_t s) {
  constexpr int BM = 32 * WM * WAVES_M, WNT = 2 * WN;
  const WsGeom w = ws_geom(M, K);
  const WeightGeom wg = weight_geom(N, K);
  const int MB = (M + BM - 1) / BM;
  const int NB = (wg.NT + WNT / 2 - 1) / (WNT / 2);
  GemmGroup g{};
  g.y[0] = act;
  g.packed[0] = gate;
  g.packed[1] = up;
  g.N[0] = g.N[1] = N;
  const int n_major = (double)M * 2.0 <= (double)N * 2.0 * 0.5625 ? 1 : 0;
  if (MB > 0xFFFF || NB > 0xFFFF) return hipErrorInvalidValue;
  const unsigned nbs = (unsigned)MB | (unsigned)NB << 16;
  const unsigned flags = (unsigned)n_major | 1u << 8 | 2u << 16;
  hipLaunchKernelGGL((gemm_f16_kernel<WAVES_M, 1, WM, WN, DEPTH, OCC, kModePair, 1, 1>),
                     dim3(((MB * NB + 7) / 8) * 8), dim3(64 * WAVES_M), 0, s,
                     reinterpret_cast<const _Float16*>(ws + w.ah_off), gate, up, nullptr, M, K, N, N, 0, nbs, 0u,
                     flags, act, reinterpret_cast<const float*>(ws + w.scale_off), nullptr, g);
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

// Tile shapes of the f16 kernel (kKernelGemmF16Tile + index names one; kKernelGemmF16 chooses).
//   0:  64 x  64, 4 wavefronts of 32 x 32, 8 stages of loads in flight
//   1: 128 x  64, 4 wavefronts of 32 x 64
//   2: 128 x 128, 4 wavefronts of 32 x 128, three workgroups per CU
//   3: 256 x 128, 4 wavefronts of 64 x 128 (each B fragment feeds two products: half the LDS reads
//      per product), loads one stage ahead only, which keeps it at 224 registers: two workgroups
//      per CU (with two stages ahead and one workgroup per CU it never beat shape 2)
//   4: 128 x  64 with one barrier per two stages (12-15 % over shape 1 at long K, 1-3 % at K = 1536; on
//      the 128 x 128 tile the same change measured no gain)
//   5: 128 x 160, 4 wavefronts of 32 x 160, two workgroups per CU: gate_proj at M = 512 is 4 x 56 = 224 of
//      these, one on almost every CU, instead of 280 tiles of 128 x 128 that leave 24 CUs with two
//      (28.8 -> 26.3 us); at M = 1024 it is 448, two per CU (41.1 -> 38.4 us)
//   6: 128 x 128, 8 wavefronts: 4 of 32 x 128 for each 32-k half of a stage (two wavefronts per SIMD from
//      a single workgroup); for 129..256 tiles, where every workgroup has a CU to itself (7-19 % over
//      shape 2). The same arrangement on the 128 x 160 tile measured 1-3 % behind shape 5.
//   7: 256 x  96, 4 wavefronts of 64 x 96, two workgroups per CU: for problems whose 256 x 128 tiles come to
//      a little more than one full round of the 512 resident workgroups (gate_proj at M = 2048: 560 tiles of
//      256 x 128 leave 48 for a second round, 752 of these cost three quarters each: 62.8 -> 57.7 us)
//   8: 256 x  96 with one barrier per two stages, one workgroup per CU: for 161..256 of these tiles, each
//      alone on its CU (gate_proj at M = 512: 188 tiles, 24.1 -> 22.2 us; o_proj and down_proj at M = 3072:
//      23.4 -> 21.4 and 96.9 -> 83.1 us; ViT fc1 and the merger at M = 1024: 20.5 -> 19.3, 62.5 -> 55.6 us).
//      With two wavefronts per SIMD from the same workgroup (k-halves) it measured the same.
//   9: 256 x 128 with one barrier per two stages: shape 3 for up to one tile per CU (3-6 % over shape 3 there:
//      gate_proj at M = 640: 26.8 -> 25.5 us; behind it as soon as two workgroups share a CU)
static hipError_t launch_f16_tile(int tile, float* y, const uint8_t* ws, const uint8_t* packed, int M,
                                  int K, int N, const GemmGroup* group, const int* group_N, int count,
                                  int ksplit, float* part, hipStream_t s) {
  switch (tile) {
    case 0:
      return launch_f16<2, 2, 1, 1, 8, 2>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 1:
      return launch_f16<4, 1, 1, 2, 2, 4>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 2:
      return launch_f16<4, 1, 1, 4, 2, 3>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 3:
      return launch_f16<4, 1, 2, 4, 1, 2>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 4:
      return launch_f16<4, 1, 1, 2, 2, 3, 2>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 5:
      return launch_f16<4, 1, 1, 5, 2, 2>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 6:
      return launch_f16<4, 1, 1, 4, 2, 2, 1, 2>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 7:
      return launch_f16<4, 1, 2, 3, 1, 2>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 8:
      return launch_f16<4, 1, 2, 3, 2, 1, 2>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
    case 9:
      return launch_f16<4, 1, 2, 4, 2, 1, 2>(y, ws, packed, M, K, N, group, group_N, count, ksplit, part, s);
  }
  return hipErrorInvalidValue;
}

// tiles: 128 x 128 tiles of the problem; tiles160: 128 x 160 tiles; tiles256: 256 x 128 tiles; tiles96: 256 x 96.
static int choose_f16_tile(long tiles, long tiles160, long tiles256, long tiles96, int K) {
  if (tiles <= 128) return 4;
  if (tiles <= 256) return 6;
  // 256 x 96 tiles, one per CU on most CUs
  if (tiles96 > 160 && tiles96 <= 256) return 8;
  // 128 x 160 tiles, two workgroups per CU: when they come to one or two per CU with few CUs left over
  const long slots = 256 * ((tiles160 + 255) / 256);
  if (tiles160 <= 512 && tiles160 * 100 >= slots * 85) return 5;
  // 256 x 128 tiles, two workgroups per CU: from three quarters of a full round on, for up to one per CU,
  // and on a long K
  if (tiles256 >= 160 && tiles256 <= 256) return 9;
  // a second round of 256 x 128 tiles that would be nearly empty: the same rows in narrower tiles
  if (tiles256 > 512 && tiles256 <= 640 && tiles96 <= 768) return 7;
  if (tiles256 >= 384 || (K >= 4096 && tiles >= 320)) return 3;
  return 2;
}

// Choice of tile shape, measured on MI355X at M = 128..8192 over the decoder and ViT shapes, by
// the number of tiles the problem has. Up to half a 128 x 128 tile per CU the 128 x 64 tile doubles the
// workgroups; up to one tile per CU the workgroup is alone on its CU and the eight-wavefront
// arrangement hides some of its latencies; a problem whose 128 x 160 tiles come to (nearly) one or two per
// CU takes those. The 256 x 128 tile reads each B fragment for two products, where LDS bandwidth bounds
// the 128-row tiles, and wins wherever its coarser tiles still fill the chip: gate_proj from M = 1536 on
// (M = 1792: 60 -> 50 us, 990 TFLOP/s; M = 8192: 253 -> 208 us, 1.08 PFLOP/s), q/o from M = 4096 on,
// down_proj from M = 3456 on; in between 128 x 128 with three resident workgroups per CU. The 64 x 64 tile
// no longer wins anywhere; it stays selectable by number.
hipError_t launch_gemm(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                       int kernel, hipStream_t s) {
  if (kernel == kKernelGemmI8) {
    return launch_gemm_i8(y, ws, packed, M, K, N, s);
  }
  if (kernel >= kKernelGemmF16Tile && kernel < kKernelGemmF16Tile + kGemmF16Tiles) {
    return launch_f16_tile(kernel - kKernelGemmF16Tile, y, ws, packed, M, K, N, nullptr, nullptr, 0, 1,
                           nullptr, s);
  }
  const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
  const long tiles160 = (long)((M + 127) / 128) * ((N + 159) / 160);
  const long tiles256 = (long)((M + 255) / 256) * ((N + 127) / 128);
  const long tiles96 = (long)((M + 255) / 256) * ((N + 95) / 96);
  return launch_f16_tile(choose_f16_tile(tiles, tiles160, tiles256, tiles96, K), y, ws, packed, M, K, N, nullptr,
                         nullptr, 0, 1, nullptr, s);
}

hipError_t launch_gemm_group(float* const* y, const uint8_t* ws, const uint8_t* const* packed,
                             const int* N, int count, int M, int K, hipStream_t s) {
  GemmGroup g{};
  long tiles = 0, tiles160 = 0, tiles256 = 0, tiles96 = 0;
  for (int i = 0; i < count; ++i) {
    g.y[i] = y[i];
    g.packed[i] = packed[i];
    g.N[i] = N[i];
    tiles += (long)((M + 127) / 128) * ((N[i] + 127) / 128);
    tiles160 += (long)((M + 127) / 128) * ((N[i] + 159) / 160);
    tiles256 += (long)((M + 255) / 256) * ((N[i] + 127) / 128);
    tiles96 += (long)((M + 255) / 256) * ((N[i] + 95) / 96);
  }
  return launch_f16_tile(choose_f16_tile(tiles, tiles160, tiles256, tiles96, K), nullptr, ws, nullptr, M, K, 0, &g, N,
                         count, 1, nullptr, s);
}

// The MLP's gate and up Linears with silu(gate) * up as the only output. Tile shape as for the two Linears
// side by side (2N columns), among the shapes whose wavefronts own whole rows of a column block pair.
hipError_t launch_gemm_pair(float* act, const uint8_t* ws, const uint8_t* gate, const uint8_t* up, int M,
                            int K, int N, hipStream_t s) {
  const long tiles = (long)((M + 127) / 128) * ((2 * N + 127) / 128);
  if (tiles <= 128) return launch_f16_pair<4, 2, 2, 4>(act, ws, gate, up, M, K, N, s);
  const long tiles256 = (long)((M + 255) / 256) * ((2 * N + 127) / 128);
  if (tiles256 >= 384 || (K >= 4096 && tiles >= 320)) {  // 256 x 128, as for a single Linear
    return launch_f16_pair<4, 4, 1, 2, 2>(act, ws, gate, up, M, K, N, s);
  }
  // 128 x (96 + 96), loads one stage ahead, two workgroups per CU: up to about a round and a half of them it
  // beats the 128 x (64 + 64) shape (N = 8960 at M = 256 / 512 / 1024: 27.2 -> 23.7, 40.6 -> 38.3, 66.3 -> 62.4 us;
  // at M = 2048 it is behind, 122 -> 140 us)
  const long tiles192 = (long)((M + 127) / 128) * ((N + 95) / 96);
  if (tiles192 <= 768) return launch_f16_pair<4, 6, 1, 2>(act, ws, gate, up, M, K, N, s);
  return launch_f16_pair<4, 4, 2, 3>(act, ws, gate, up, M, K, N, s);
}

// Split-K: tile shape and number of parts for a problem (parts == 1: not worth splitting).
// Measured on MI355X (down_proj, K = 8960, N = 1536): M = 128: 44 -> 16 us, 256: 44 -> 21,
// 512: 47 -> 29, 1024: 50 -> 45, 2048: 85 -> 82; at K = 1536 and K = 5120 the second kernel and the
// partial sums' traffic cost what the shorter loops gain, so only long K qualifies. Parts: about one or
// two workgroups per CU in all (10 parts up to 24 tiles, 5 up to 96, then 4); more parts only add
// partial sums for the second kernel to read.
SplitPlan splitk_plan(int M, int K, int N) {
  SplitPlan p{2, 1};
  const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
  const int nstages = (K + kF16BK - 1) / kF16BK;
  if (M <= kGemvMaxM || nstages < 96 || tiles > 256) return p;
  p.parts = tiles <= 24 ? 10 : tiles <= 96 ? 5 : 4;
  if (tiles <= 16) {
    p.tile = 1;  // 128 x 64: twice the workgroups (M = 128: 19 -> 16 us)
  } else if (tiles * p.parts <= 256) {
    p.tile = 6;  // every workgroup alone on its CU: the eight-wavefront shape (M = 512: 30.1 -> 29.1 us)
  }
  return p;
}

// y == nullptr: no reduction; part[i][M][N], i < parts, then holds sums that already carry the row and column
// factors, for a reader that computes (((part[0] + part[1]) + ...) + bias) itself.
hipError_t launch_gemm_splitk(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                              float* part, hipStream_t s) {
  const SplitPlan p = splitk_plan(M, K, N);
  return launch_f16_tile(p.tile, y, ws, packed, M, K, N, nullptr, nullptr, 0, p.parts, part, s);
}

const float* linear_bias(const uint8_t* packed, int N, int K) {
  return reinterpret_cast<const float*>(packed + weight_geom(N, K).bias_off);
}

}  // namespace w4
