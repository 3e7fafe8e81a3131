// Prefill attention with its two products on the 16-bit matrix pipe at f32 accuracy: every f32 operand is
// split into three bf16 terms, x = x1 + x2 + x3 (each the truncation of what is left: 24 significant bits
// in all, the exponent range of f32), and a product x y is evaluated as the six partial products
// x1 y1 + x1 y2 + x2 y1 + x1 y3 + x3 y1 + x2 y2 (what is left out is below 2^-23 of |x y|), each a
// v_mfma_f32_32x32x16_bf16 that accumulates in f32. A 32 x 32 (query, key) block pair then costs a SIMD
// 96 x 32 = 3072 clocks instead of the 8192 of v_mfma_f32_32x32x2_f32; the longest query block of a
// 512-token prompt (16 pairs on a CU's four SIMDs) bounds the launch at 12 k clocks instead of 33 k.
//
// Same operator as attention_prefill_mfma_kernel (w4a32_glue.hip): out[m][h] = softmax(q[m][h] . K[0..pos0+m]
// / sqrt(128)) V, QWenAttention::forward, mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:133-151 (matmul,
// CausalMaskOp.cpp:22-71, SoftmaxOp.cpp:18-50, matmul). Two launches:
//
//   split_kv_kernel     K and V rows of keys [0, n_keys) -> their bf16 terms in scratch, once per call instead of
//                       once per query block, as the operands the second launch loads: per (kv head, block of
//                       32 keys) 24 KB of K operands and 24 KB of V operands, each operand (8 bf16 per lane, 1 KB
//                       per wavefront) contiguous in lane order, so that every operand load is one coalesced
//                       1 KB read (as rows with the keys or dims of a lane 768 or 2 KP bytes apart, a load touched
//                       32 cache lines and used a quarter of each: the V loads alone were a third of the time):
//                         K operand (k-step s, term t):    lane (h, j) = key j, dims 16 s + 8 h .. + 7
//                         V operand (term t, dim block c, k-step ks): lane (h, j) = dim 32 c + j, keys at positions
//                             16 ks + 8 h .. + 7 of the block, where position 8 h' + e of a group of 16 keys holds
//                             key 8 (e / 4) + 4 h' + e % 4: the order the first product's result registers have,
//                             so the softmaxed scores go from the accumulator to the next product's operand
//                             without a cross-lane move (V transposed: the second product runs over keys).
//                       Keys past the last one of a 32-key block are written as zeros (a zero weight times
//                       whatever the cache holds there must not reach the sums).
//   attention16_kernel  workgroup = (head, 32 queries); its wavefronts take the 32-key blocks round-robin and
//                       merge through LDS, as in the f32 kernel. Both products transposed, so a lane stands for
//                       one query and the online-softmax state is per lane:
//                         S^T = K Q^T     A = K terms (lane: key l % 32, dims 16 s + 8 (l / 32) ..), B = Q terms
//                                         from LDS (split once per workgroup)
//                         O^T += V^T P^T  A = V^T terms, B = the terms of the softmaxed S^T registers
#include "w4a32_decoder.h"
#include "w4a32_internal.h"

namespace w4 {

namespace {

constexpr int kHd = 128;  // head_dim
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));

// bf16 terms of x (bits in the high half of each result): truncations, so every remainder is exact
__device__ __forceinline__ void split3(float x, uint32_t& t1, uint32_t& t2, uint32_t& t3) {
  t1 = __float_as_uint(x) & 0xFFFF0000u;
  const float r1 = x - __uint_as_float(t1);
  t2 = __float_as_uint(r1) & 0xFFFF0000u;
  const float r2 = r1 - __uint_as_float(t2);
  t3 = __float_as_uint(r2) & 0xFFFF0000u;
}
// two terms (high halves) -> one dword of two bf16, `lo` first in memory
__device__ __forceinline__ uint32_t pack2(uint32_t lo, uint32_t hi) { return (lo >> 16) | hi; }

// 8 consecutive f32 -> three operands of 8 bf16
__device__ __forceinline__ void split3x8(const float (&x)[8], uint4 (&out)[3]) {
  uint32_t t[3][8];
#pragma unroll
  for (int e = 0; e < 8; ++e) split3(x[e], t[0][e], t[1][e], t[2][e]);
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    out[k] = make_uint4(pack2(t[k][0], t[k][1]), pack2(t[k][2], t[k][3]), pack2(t[k][4], t[k][5]),
                        pack2(t[k][6], t[k][7]));
  }
}

__device__ __forceinline__ v16f mfma16(uint4 a, uint4 b, v16f c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), c, 0, 0, 0);
}
// position inside a group of 16 keys at which the V operands keep key offset o (see the file header)
__device__ __forceinline__ int vt_pos(int o) { return 8 * ((o >> 2) & 1) + 4 * (o >> 3) + (o & 3); }

constexpr int kOpBytes = 64 * 16;             // one operand: 16 bytes per lane
constexpr int kBlkBytes = 24 * kOpBytes;      // the 24 K operands (or the 24 V operands) of a block of 32 keys
__device__ __forceinline__ int k_op(int s, int t) { return s * 3 + t; }
__device__ __forceinline__ int v_op(int t, int c, int ks) { return (t * 4 + c) * 2 + ks; }

// K operands of one 32-key block: called by 256 threads, thread = (key_l = t / 8, sstep = t % 8) holds the 16
// dims of k-step sstep of key key_l, which are the two halves (h = 0, 1) of lane key_l of that k-step's operands.
__device__ __forceinline__ void store_k_operands(const float (&kx)[16], int key_l, int sstep,
                                                 uint8_t* __restrict__ kblk) {
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    float x8[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) x8[e] = kx[8 * half + e];
    uint4 terms[3];
    split3x8(x8, terms);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      *reinterpret_cast<uint4*>(kblk + (size_t)k_op(sstep, k) * kOpBytes + (32 * half + key_l) * 16) = terms[k];
    }
  }
}

// V^T operands of one 32-key block, read transposed: called by 256 threads, thread = (dim d = t % 128, h = t / 128)
// is lane (h, d % 32) of the operands of dim block d / 32; for k-step ks it holds the block's keys
// 16 ks + 4 h + {0, 1, 2, 3, 8, 9, 10, 11} (positions 16 ks + 8 h .. + 7 in operand order, see the file header).
// The 64 lanes of a load are 64 consecutive dims of one key: one coalesced 256-byte read; nothing goes through
// LDS. `row(key_in_block)` returns the address of that key's V row (any valid row for a key past the last one) and
// `keep(key_in_block, d, x)` the value to use (0 past the last key; it may append x to the cache). All 16 loads
// are issued before the first result is looked at.
template <typename Row, typename Keep>
__device__ __forceinline__ void store_v_operands(Row row, Keep keep, uint8_t* __restrict__ vblk) {
  const int d = threadIdx.x & 127, h = threadIdx.x >> 7;
  float x[2][8];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int e = 0; e < 8; ++e) x[ks][e] = row(16 * ks + 4 * h + 8 * (e >> 2) + (e & 3))[d];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int e = 0; e < 8; ++e) x[ks][e] = keep(16 * ks + 4 * h + 8 * (e >> 2) + (e & 3), d, x[ks][e]);
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    uint4 terms[3];
    split3x8(x[ks], terms);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      *reinterpret_cast<uint4*>(vblk + (size_t)v_op(k, d >> 5, ks) * kOpBytes + (32 * h + (d & 31)) * 16) = terms[k];
    }
  }
}

__device__ __forceinline__ void load16(const float* __restrict__ src, float (&x)[16]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float4 a = *reinterpret_cast<const float4*>(src + 4 * i);
    x[4 * i] = a.x; x[4 * i + 1] = a.y; x[4 * i + 2] = a.z; x[4 * i + 3] = a.w;
  }
}
__device__ __forceinline__ void store16(float* __restrict__ dst, const float (&x)[16]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    *reinterpret_cast<float4*>(dst + 4 * i) = make_float4(x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]);
  }
}

// grid (key blocks of 32, 2 * kv heads), 256 threads: blockIdx.y < Hkv writes the K operands of a block,
// the others its V^T operands
__global__ __launch_bounds__(256) void split_kv_kernel(const float* __restrict__ kc, const float* __restrict__ vc,
                                                       uint8_t* __restrict__ ks, uint8_t* __restrict__ vts,
                                                       int n_keys, int max_seq, int NKB, int Hkv) {
  const int kb = blockIdx.x;
  if ((int)blockIdx.y < Hkv) {
    const int hk = blockIdx.y;
    const int key_l = threadIdx.x >> 3, sstep = threadIdx.x & 7;
    const int key = 32 * kb + key_l;
    float kx[16];
    load16(kc + ((size_t)hk * max_seq + (key < n_keys ? key : 0)) * kHd + 16 * sstep, kx);
    if (key >= n_keys) {
#pragma unroll
      for (int i = 0; i < 16; ++i) kx[i] = 0.0f;
    }
    store_k_operands(kx, key_l, sstep, ks + ((size_t)hk * NKB + kb) * kBlkBytes);
    return;
  }
  const int hk = blockIdx.y - Hkv;
  const float* vrow = vc + (size_t)hk * max_seq * kHd;
  store_v_operands(
      [&](int kl) {
        const int key = 32 * kb + kl;  // wavefront-uniform
        return vrow + (size_t)(key < n_keys ? key : 0) * kHd;
      },
      [&](int kl, int, float x) { return 32 * kb + kl < n_keys ? x : 0.0f; },
      vts + ((size_t)hk * NKB + kb) * kBlkBytes);
}

// rope_kv_kernel (w4a32_glue.hip) and split_kv_kernel in one launch, for a prefill that runs attention16_kernel
// next: grid (key blocks of 32, 2 * Hkv + Hq), 256 threads.
//   blockIdx.y <  Hkv:     the K operands of kv head blockIdx.y. A key below pos0 comes from the cache as it is;
//                          key pos0 + m is row m of k, rotated here (the arithmetic of rope_kv_kernel) and also
//                          appended to the cache; keys from n_keys on are zeros.
//   blockIdx.y <  2 Hkv:   the V^T operands likewise (row m of v, appended to the cache).
//   otherwise:             rotates rows 32 blockIdx.x .. + 31 of query head blockIdx.y - 2 Hkv in place; a thread
//                          owns dims 8 i .. 8 i + 7 and their partners 64 + 8 i .. (nobody else reads what it
//                          writes).
__global__ __launch_bounds__(256) void rope_split_kv_kernel(
    float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ sin_t, const float* __restrict__ cos_t, float* __restrict__ kc,
    float* __restrict__ vc, uint8_t* __restrict__ ks, uint8_t* __restrict__ vts, int M, int Hq, int Hkv,
    int pos0, int max_seq, int NKB) {
  constexpr int kHalf = kHd / 2;
  const int kb = blockIdx.x;
  const int row_l = threadIdx.x >> 3, sstep = threadIdx.x & 7;
  const int n_keys = pos0 + M;
  if ((int)blockIdx.y >= 2 * Hkv) {
    const int h = blockIdx.y - 2 * Hkv, m = 32 * kb + row_l;
    if (m >= M) return;
    float* x = q + ((size_t)m * Hq + h) * kHd + 8 * sstep;
    const float* st = sin_t + (size_t)(pos0 + m) * kHalf + 8 * sstep;
    const float* ct = cos_t + (size_t)(pos0 + m) * kHalf + 8 * sstep;
    const float4 a0 = *reinterpret_cast<const float4*>(x), a1 = *reinterpret_cast<const float4*>(x + 4);
    const float4 b0 = *reinterpret_cast<const float4*>(x + kHalf), b1 = *reinterpret_cast<const float4*>(x + kHalf + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(st), s1 = *reinterpret_cast<const float4*>(st + 4);
    const float4 c0 = *reinterpret_cast<const float4*>(ct), c1 = *reinterpret_cast<const float4*>(ct + 4);
    const float x0[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    const float x1[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
    const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    float y0[8], y1[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      y0[e] = x0[e] * cs[e] - x1[e] * sn[e];
      y1[e] = x0[e] * sn[e] + x1[e] * cs[e];
    }
    *reinterpret_cast<float4*>(x) = make_float4(y0[0], y0[1], y0[2], y0[3]);
    *reinterpret_cast<float4*>(x + 4) = make_float4(y0[4], y0[5], y0[6], y0[7]);
    *reinterpret_cast<float4*>(x + kHalf) = make_float4(y1[0], y1[1], y1[2], y1[3]);
    *reinterpret_cast<float4*>(x + kHalf + 4) = make_float4(y1[4], y1[5], y1[6], y1[7]);
    return;
  }
  if ((int)blockIdx.y >= Hkv) {
    const int hk = blockIdx.y - Hkv;
    float* vcache = vc + (size_t)hk * max_seq * kHd;
    store_v_operands(
        [&](int kl) {
          const int key = 32 * kb + kl;  // wavefront-uniform
          const float* cached = vcache + (size_t)(key < pos0 ? key : 0) * kHd;
          const float* fresh = v + ((size_t)(key >= pos0 && key < n_keys ? key - pos0 : 0) * Hkv + hk) * kHd;
          return key < pos0 ? cached : fresh;
        },
        [&](int kl, int d, float x) {
          const int key = 32 * kb + kl;
          if (key >= n_keys) return 0.0f;
          if (key >= pos0) vcache[(size_t)key * kHd + d] = x;
          return x;
        },
        vts + ((size_t)hk * NKB + kb) * kBlkBytes);
    return;
  }
  const int hk = blockIdx.y, d0 = 16 * sstep;
  const int key = 32 * kb + row_l;
  float kx[16];
  if (key >= n_keys) {
#pragma unroll
    for (int i = 0; i < 16; ++i) kx[i] = 0.0f;
  } else if (key < pos0) {
    load16(kc + ((size_t)hk * max_seq + key) * kHd + d0, kx);
  } else {
    const size_t src = ((size_t)(key - pos0) * Hkv + hk) * kHd;
    // this thread's 16 dims and their partners in the other half of the head vector
    const int dp = d0 < kHalf ? d0 + kHalf : d0 - kHalf, dt = d0 < kHalf ? d0 : d0 - kHalf;
    float own[16], par[16], sn[16], cs[16];
    load16(k + src + d0, own);
    load16(k + src + dp, par);
    load16(sin_t + (size_t)key * kHalf + dt, sn);
    load16(cos_t + (size_t)key * kHalf + dt, cs);
    if (d0 < kHalf) {
#pragma unroll
      for (int i = 0; i < 16; ++i) kx[i] = own[i] * cs[i] - par[i] * sn[i];
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) kx[i] = par[i] * sn[i] + own[i] * cs[i];
    }
    store16(kc + ((size_t)hk * max_seq + key) * kHd + d0, kx);
  }
  store_k_operands(kx, row_l, sstep, ks + ((size_t)hk * NKB + kb) * kBlkBytes);
}

template <int kWaves>
__global__ __launch_bounds__(64 * kWaves) void attention16_kernel(
    const float* __restrict__ q, const uint8_t* __restrict__ ks, const uint8_t* __restrict__ vts,
    float* __restrict__ out, int M, int Hq, int Hkv, int NKB, int pos0, float scale) {
  extern __shared__ __align__(16) uint8_t smem16[];
  uint4* s_q = reinterpret_cast<uint4*>(smem16);                          // [8 k-steps][3 terms][64 lanes]
  float* s_merge = reinterpret_cast<float*>(smem16 + 8 * 3 * 64 * 16);     // [kWaves - 1][66][64]
  const int h = blockIdx.x, qb = blockIdx.y;
  const int hk = h / (Hq / Hkv);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int j = lane & 31, hh = lane >> 5;

  const int m_q = min(32 * qb + j, M - 1);           // this lane's query row (rows past M repeat the last)
  const int q_pos = pos0 + m_q;                        // its position: it sees keys 0..q_pos
  const int last_key = pos0 + min(32 * qb + 31, M - 1);
  const int nkb = last_key / 32 + 1;                   // key blocks this query block touches

  // Q^T operands of the workgroup's 32 queries, split once: item (k-step s, lane) = dims 16 s + 8 hh .. + 7 of
  // query j
  for (int it = threadIdx.x; it < 8 * 64; it += 64 * kWaves) {
    const int s = it >> 6, l = it & 63;
    const int mq = min(32 * qb + (l & 31), M - 1);
    const float* src = q + ((size_t)mq * Hq + h) * kHd + 16 * s + 8 * (l >> 5);
    const float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
    const float x8[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint4 terms[3];
    split3x8(x8, terms);
#pragma unroll
    for (int k = 0; k < 3; ++k) s_q[(s * 3 + k) * 64 + l] = terms[k];
  }
  __syncthreads();

  const uint8_t* kbase = ks + (size_t)hk * NKB * kBlkBytes + 16 * lane;
  const uint8_t* vbase = vts + (size_t)hk * NKB * kBlkBytes + 16 * lane;

  v16f o[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[c][v] = 0.0f;
  float run_max = -INFINITY, run_sum = 0.0f;

  // One wavefront per SIMD with every operand of a block requested a phase ahead: the K terms of a wavefront's
  // next block while the current one's softmax and second product run, the V terms of the current block at its
  // start, under the first product. (A CU's vector L1 delivers 64 bytes a clock, and a block's 48 KB of operands
  // per wavefront are about what the four SIMDs' 3072 product clocks leave room for: loads that wait for their
  // use cost more than the matrix pipe saves - with operands requested just before their products the kernel
  // measured slower than the f32 one.)
  uint4 kop[8][3];
  auto load_k = [&](int kb) {
    const uint8_t* blk = kbase + (size_t)kb * kBlkBytes;
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int k = 0; k < 3; ++k) kop[s][k] = *reinterpret_cast<const uint4*>(blk + k_op(s, k) * kOpBytes);
  };
  if (wave < nkb) load_k(wave);
  for (int kb = wave; kb < nkb; kb += kWaves) {
    // V^T operands [c][ks][term] of this block
    uint4 vop[4][2][3];
    {
      const uint8_t* blk = vbase + (size_t)kb * kBlkBytes;
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int ksx = 0; ksx < 2; ++ksx)
#pragma unroll
          for (int k = 0; k < 3; ++k) vop[c][ksx][k] = *reinterpret_cast<const uint4*>(blk + v_op(k, c, ksx) * kOpBytes);
    }
    // S^T block. Two accumulators (even and odd k-steps) whose products alternate: a product that accumulates
    // into the result of the one just before it waits for that result (about twice the issue time).
    v16f st, st1;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      st[v] = 0.0f;
      st1[v] = 0.0f;
    }
#pragma unroll
    for (int s = 0; s < 8; s += 2) {
      uint4 q0[3], q1[3];
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        q0[k] = s_q[(s * 3 + k) * 64 + lane];
        q1[k] = s_q[((s + 1) * 3 + k) * 64 + lane];
      }
      // the six partial products, smallest first
      st = mfma16(kop[s][1], q0[1], st);
      st1 = mfma16(kop[s + 1][1], q1[1], st1);
      st = mfma16(kop[s][2], q0[0], st);
      st1 = mfma16(kop[s + 1][2], q1[0], st1);
      st = mfma16(kop[s][0], q0[2], st);
      st1 = mfma16(kop[s + 1][0], q1[2], st1);
      st = mfma16(kop[s][1], q0[0], st);
      st1 = mfma16(kop[s + 1][1], q1[0], st1);
      st = mfma16(kop[s][0], q0[1], st);
      st1 = mfma16(kop[s + 1][0], q1[1], st1);
      st = mfma16(kop[s][0], q0[0], st);
      st1 = mfma16(kop[s + 1][0], q1[0], st1);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) st[v] += st1[v];
    __builtin_amdgcn_sched_barrier(0);
    if (kb + kWaves < nkb) load_k(kb + kWaves);  // the next block's K terms, into the registers just used
    __builtin_amdgcn_sched_barrier(0);
    // causal mask, online softmax (a query's 32 scores of the block sit in lanes j and j + 32)
    float blk_max = -INFINITY;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int key = 32 * kb + 8 * (v >> 2) + 4 * hh + (v & 3);
      st[v] = key <= q_pos ? st[v] * scale : -INFINITY;
      blk_max = fmaxf(blk_max, st[v]);
    }
    blk_max = fmaxf(blk_max, __shfl_xor(blk_max, 32, 64));
    const float new_max = fmaxf(run_max, blk_max);
    // new_max = -inf only while every key so far was masked for this query: all weights 0
    const float corr = run_max == -INFINITY ? 0.0f : __expf(run_max - new_max);
    float psum = 0.0f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      st[v] = st[v] == -INFINITY ? 0.0f : __expf(st[v] - new_max);
      psum += st[v];
    }
    psum += __shfl_xor(psum, 32, 64);
    run_sum = run_sum * corr + psum;
    run_max = new_max;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[c][v] *= corr;
    // P^T operands: registers 8 ks .. 8 ks + 7 are the 8 k-values of k-step ks as they are
    uint4 pop[2][3];
#pragma unroll
    for (int ksx = 0; ksx < 2; ++ksx) {
      float x8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) x8[e] = st[8 * ksx + e];
      split3x8(x8, pop[ksx]);
    }
    // O^T += V^T P^T
    // (the four dim blocks' accumulators take turns, see above)
#pragma unroll
    for (int ksx = 0; ksx < 2; ++ksx) {
      constexpr int kA[6] = {1, 2, 0, 1, 0, 0}, kB[6] = {1, 0, 2, 0, 1, 0};  // the six partial products
#pragma unroll
      for (int p = 0; p < 6; ++p)
#pragma unroll
        for (int c = 0; c < 4; ++c) o[c] = mfma16(vop[c][ksx][kA[p]], pop[ksx][kB[p]], o[c]);
    }
  }

  // wavefronts 1.. hand their (max, sum, O^T) to wavefront 0
  if (wave > 0) {
    float* dst = s_merge + (size_t)(wave - 1) * 66 * 64 + lane;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) dst[(16 * c + v) * 64] = o[c][v];
    dst[64 * 64] = run_max;
    dst[65 * 64] = run_sum;
  }
  __syncthreads();
  if (wave > 0) return;
  float wmax[kWaves - 1], wsum[kWaves - 1];
  float total_max = run_max;
#pragma unroll
  for (int w = 0; w < kWaves - 1; ++w) {
    wmax[w] = s_merge[(size_t)w * 66 * 64 + 64 * 64 + lane];
    wsum[w] = s_merge[(size_t)w * 66 * 64 + 65 * 64 + lane];
    total_max = fmaxf(total_max, wmax[w]);
  }
  const float own_w = run_max == -INFINITY ? 0.0f : __expf(run_max - total_max);
  float total_sum = run_sum * own_w;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[c][v] *= own_w;
#pragma unroll
  for (int w = 0; w < kWaves - 1; ++w) {
    const float wt = wmax[w] == -INFINITY ? 0.0f : __expf(wmax[w] - total_max);
    total_sum += wsum[w] * wt;
    const float* src = s_merge + (size_t)w * 66 * 64 + lane;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[c][v] += src[(16 * c + v) * 64] * wt;
  }
  // lane = query; register v of block c = dim 32 c + 8 (v / 4) + 4 hh + v % 4: four registers -> one float4
  if (32 * qb + j < M) {
    const float inv = 1.0f / total_sum;  // every query sees at least its own key
    float* dst = out + ((size_t)(32 * qb + j) * Hq + h) * kHd;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        *reinterpret_cast<float4*>(dst + 32 * c + 8 * g4 + 4 * hh) = make_float4(
            o[c][4 * g4] * inv, o[c][4 * g4 + 1] * inv, o[c][4 * g4 + 2] * inv, o[c][4 * g4 + 3] * inv);
      }
  }
}

}  // namespace

// bytes of the K and V operands for n_keys keys
size_t attention16_scratch_bytes(int n_keys, int Hkv) {
  return 2 * (size_t)Hkv * ((n_keys + 31) / 32) * kBlkBytes;
}

static hipError_t launch_attention16_products(const float* q, const uint8_t* ks, const uint8_t* vts, float* out,
                                              int M, int Hq, int Hkv, int NKB, int pos0, hipStream_t s) {
  const float scale = 1.0f / sqrtf((float)kHd);
  constexpr size_t kQBytes = 8 * 3 * 64 * 16;
  constexpr int W = 4;  // one wavefront per SIMD: its operand prefetch takes most of the register file
  const size_t lds = kQBytes + sizeof(float) * (W - 1) * 66 * 64;
  static LdsLimitOnce raised;  // above the default limit of dynamic LDS
  if (hipError_t e = raised.raise(reinterpret_cast<const void*>(attention16_kernel<W>), lds); e != hipSuccess) return e;
  hipLaunchKernelGGL((attention16_kernel<W>), dim3(Hq, (M + 31) / 32), dim3(64 * W), lds, s, q, ks, vts, out, M, Hq,
                     Hkv, NKB, pos0, scale);
  return hipGetLastError();
}

hipError_t launch_attention16(const float* q, const float* kc, const float* vc, float* out, int M, int Hq, int Hkv,
                              int max_seq, int pos0, uint8_t* scratch, hipStream_t s) {
  const int n_keys = pos0 + M;
  const int NKB = (n_keys + 31) / 32;
  uint8_t* ks = scratch;
  uint8_t* vts = scratch + (size_t)Hkv * NKB * kBlkBytes;
  hipLaunchKernelGGL(split_kv_kernel, dim3(NKB, 2 * Hkv), dim3(256), 0, s, kc, vc, ks, vts, n_keys, max_seq, NKB, Hkv);
  if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  return launch_attention16_products(q, ks, vts, out, M, Hq, Hkv, NKB, pos0, s);
}

hipError_t launch_rope_attention16(float* q, const float* k, const float* v, const float* sin_t,
                                   const float* cos_t, float* kc, float* vc, float* out, int M, int Hq, int Hkv,
                                   int max_seq, int pos0, uint8_t* scratch, hipStream_t s) {
  const int n_keys = pos0 + M;
  const int NKB = (n_keys + 31) / 32;
  uint8_t* ks = scratch;
  uint8_t* vts = scratch + (size_t)Hkv * NKB * kBlkBytes;
  hipLaunchKernelGGL(rope_split_kv_kernel, dim3(NKB, 2 * Hkv + Hq), dim3(256), 0, s, q, k, v, sin_t, cos_t, kc, vc, ks,
                     vts, M, Hq, Hkv, pos0, max_seq, NKB);
  if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  return launch_attention16_products(q, ks, vts, out, M, Hq, Hkv, NKB, pos0, s);
}

}  // namespace w4
