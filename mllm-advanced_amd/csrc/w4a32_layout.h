// Device data layouts of the W4A32 Linear on MI355X, shared by host and kernels.
//
// WEIGHT BLOB ("tiles | rsum | bias"), for an [N][K] Linear, K % 32 == 0:
//
//   Np = N rounded up to 16, Kp = K rounded up to 128 (padding holds q = 0, scale = +0).
//   tiles: tile (nt, kc) covers rows 16*nt .. +15 and k 128*kc .. +127 (four scale blocks)
//          and occupies kTileBytes = 1152 contiguous bytes at ((nt * KC) + kc) * 1152:
//
//     [0, 1024)    64 lanes x 16 B. Lane l = 16*g + j  (g = k-group 0..3, j = row in tile)
//                  holds four dwords; dword d belongs to scale block 4*kc + d and carries the
//                  8 weights of row 16*nt + j at k = 128*kc + 32*d + 8*g + (0..7).
//                  One wavefront-wide 128-bit load therefore reads 1 KiB contiguous, and
//                  dword d of all 64 lanes is exactly the B operand of one 16x16x32 MFMA
//                  (n = j, k-slice = g) that stays inside ONE scale block.
//                  Inside a dword, nibble position 2e holds k offset e, position 2e+1 holds
//                  k offset 4+e (e = 0..3), each as 4-bit two's complement of q = u4 - 8.
//                  So (w << 4) & 0xF0F0F0F0 are the int8 values 16*q of k offsets 0..3 and
//                  w & 0xF0F0F0F0 those of offsets 4..7: two ops per 8 weights, no sign fix.
//     [1024, 1152) 16 rows x 4 bf16 scales: scale of (row j, block 4*kc + d) at 1024 + 8*j + 2*d.
//
//   rsum:  f32 [Np] at tiles_bytes: sum_b f32(scale_b) * (float)(sum_{k in b} q), accumulated
//          in block order. Lets the int8 kernels add the activation offset once per output:
//          sum_k (a_q + off) q s = sum_k a_q q s + off * rsum.
//   bias:  f32 [Np] after rsum (zeros when the layer has none).
//   rowmul: f32 [Np] after bias: 2^E_n, where E_n puts the row's largest |scale| in [2^11, 2^12).
//   hscale: per tile 64 x f16 (128 B, same order as the bf16 scales in the tile) after rowmul:
//          scale * 2^-E_n. A bf16 scale has 8 significant bits, so this is exact whenever it is
//          a normal f16, i.e. for every block whose scale is within 2^-25 of the row's largest;
//          then q * hscale (4 + 8 bits) is exact in f16 too. The f16 MFMA prefill kernel uses
//          this plane and multiplies its f32 accumulators by rowmul.
//
// ACTIVATION WORKSPACE for M rows (Mp = M rounded up to 32):
//
//   [0, 4*Mp)            f32  recip_scale[m]   (the "lhs scale" applied to the output)
//   [4*Mp, 8*Mp)         i32  neg_zp[m]        (the "lhs offset" = -zero_point)
//   hdr = round_up(8*Mp, 256)
//   [hdr, hdr + Mp*K)    i8   a_q[m][k] row-major
//   then, 256-aligned    f16  a_h = (a_q + neg_zp) exactly (|.| <= 255), only written when M > 8,
//                        stored as 2 KiB chunks so that the f16 MFMA kernel reads whole
//                        chunks instead of 32 rows lying K*2 bytes apart:
//                          chunk (mt, kb) = rows 32*mt..+31, k 32*kb..+31, at
//                          (mt * K/32 + kb) * 2048, row-major inside: row i at i*64, its four
//                          groups of 8 k at 16 bytes each; inside a group the order is
//                          k0,k2,k4,k6,k1,k3,k5,k7 - the order in which a weight tile dword
//                          unpacks to f16 pairs (see kHalfOrder).
#pragma once

#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define W4_HD __host__ __device__ inline
#else
#define W4_HD inline
#endif

namespace w4 {

constexpr int kBlockLen = 32;
constexpr int kTileRows = 16;
constexpr int kTileK = 128;
constexpr int kTileQBytes = 1024;
constexpr int kTileScaleBytes = 128;
constexpr int kTileBytes = kTileQBytes + kTileScaleBytes;
constexpr int kGemvMaxM = 8;

W4_HD int round_up(int v, int m) { return (v + m - 1) / m * m; }
W4_HD size_t round_up_sz(size_t v, size_t m) { return (v + m - 1) / m * m; }

struct WeightGeom {
  int N, K, Np, Kp, NT, KC;
  size_t tiles_bytes, rsum_off, bias_off, rowmul_off, hscale_off, total_bytes;
};

W4_HD WeightGeom weight_geom(int N, int K) {
  WeightGeom g;
  g.N = N;
  g.K = K;
  g.Np = round_up(N, kTileRows);
  g.Kp = round_up(K, kTileK);
  g.NT = g.Np / kTileRows;
  g.KC = g.Kp / kTileK;
  g.tiles_bytes = (size_t)g.NT * g.KC * kTileBytes;
  g.rsum_off = g.tiles_bytes;
  g.bias_off = g.rsum_off + (size_t)g.Np * 4;
  g.rowmul_off = g.bias_off + (size_t)g.Np * 4;
  g.hscale_off = g.rowmul_off + (size_t)g.Np * 4;
  g.total_bytes = g.hscale_off + (size_t)g.NT * g.KC * kTileScaleBytes;
  return g;
}

struct WsGeom {
  int M, K, Mp;
  size_t scale_off, off_off, aq_off, ah_off, total_bytes;
};

W4_HD WsGeom ws_geom(int M, int K) {
  WsGeom g;
  g.M = M;
  g.K = K;
  g.Mp = round_up(M, 32);
  g.scale_off = 0;
  g.off_off = (size_t)4 * g.Mp;
  g.aq_off = round_up_sz((size_t)8 * g.Mp, 256);
  g.ah_off = g.aq_off + round_up_sz((size_t)g.Mp * K, 256);
  g.total_bytes = g.ah_off + (M > kGemvMaxM ? (size_t)g.Mp * K * 2 : 0);
  return g;
}

// Nibble position (0..7) inside a tile dword of the weight at k offset e (0..7) in its 8-group.
W4_HD int nibble_pos(int e) { return e < 4 ? 2 * e : 2 * (e - 4) + 1; }

// Masking a tile dword with 0x000F000F after shifting right by 0, 4, 8, 12 bits yields the
// nibble pairs (0,4), (1,5), (2,6), (3,7) = k offsets (0,2), (4,6), (1,3), (5,7).
// kHalfOrder[i] is the k offset stored at position i of an 8-group of a_h.
constexpr int kHalfOrder[8] = {0, 2, 4, 6, 1, 3, 5, 7};

}  // namespace w4
