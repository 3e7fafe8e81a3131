// The f32 operators a Qwen2-style decoder runs between its quantized Linears: embedding gather,
// RMSNorm (optionally with the residual add in front), RoPE + KV-cache append, attention over the
// cache, SiLU*mul, residual add, greedy argmax. All of them are small, latency-bound kernels at
// decode sizes; the point of having them here is that a whole token runs on the device without a
// host round trip and can be replayed from a HIP graph (positions and lengths are read from
// device memory, never baked into the launch).
//
// Reference behaviour followed (file:line in the reference tree):
//   RMSNorm     mllm/Backends/Arm/Ops/RMSNormOp.cpp:36-76     y = x * (w * 1/sqrt(mean(x^2) + eps))
//   RoPE        mllm/Backends/Arm/Kernels/rope.cpp:20-80      half-split pairs (d, d + D/2),
//               theta_d = pos / base^(2d/D), y0 = x0 c - x1 s, y1 = x0 s + x1 c
//   KV cache    mllm/Backends/Arm/Ops/KVCacheOp.cpp:44-72     append at the current length; the
//               reference stores every KV head `repeat` times, here a query head indexes its KV head
//   attention   mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:133-151  softmax(q k^T / sqrt(D)) v,
//               query at position p sees keys 0..p (CausalMaskOp.cpp:22-71, SoftmaxOp.cpp:18-50)
//   SiLU * mul  modeling_ds_qwen2.hpp:47-54
//   embedding   mllm/Backends/Arm/Ops/LLMEmbeddingTokenOp.cpp:24-50 (int64 ids, f32 rows)
//   argmax      mllm/Models/AutoLLM.hpp:70-88 (strict '>': the first maximum wins)
#include "w4a32_internal.h"

namespace w4 {

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Sum over the workgroup (blockDim.x a multiple of 64, at most 1024); every thread gets the total.
__device__ __forceinline__ float block_sum(float v, float* s_part) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if ((threadIdx.x & 63) == 0) s_part[wave] = v;
  __syncthreads();
  float t = 0.0f;
  for (int w = 0; w < nw; ++w) t += s_part[w];
  __syncthreads();
  return t;
}

// Partial results that another workgroup of the same launch will read. The L2s of the XCDs are not
// coherent with each other for plain accesses, and an agent-scope fence pays for that with a
// write-back / invalidate of the whole cache; a device-scope store or load of just these words
// goes to the coherence point directly.
__device__ __forceinline__ void store_shared_across_wgs(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_shared_across_wgs(int* p, int v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_shared_across_wgs(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int load_shared_across_wgs(const int* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Hand-over of partial results to the last workgroup to arrive at a counter.
// Writer: stores_done() after the device-scope stores and before the barrier / counter increment. A
// workgroup-scope release fence alone does not have to wait for global stores that are still in flight,
// so the wait is written out: on gfx9 stores count in vmcnt, and a device-scope (write-through) store is
// acknowledged once it has reached the coherence point. After it every store this wavefront issued above
// is visible to device-scope loads of any workgroup; the fence keeps the compiler from moving memory
// accesses across it. No cache write-back or invalidate is involved.
// Reader: the workgroup whose increment returns the last ticket calls arrivals_seen() before its
// device-scope loads (which bypass the non-coherent cache levels); it only pins the order for the compiler,
// the hardware issues a wavefront's memory instructions in program order behind the returned atomic.
__device__ __forceinline__ void stores_done() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}
__device__ __forceinline__ void arrivals_seen() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}
}  // namespace

// ---------------------------------------------------------------------------------------------
// Embedding gather: out[m][:] = table[ids[m]][:]
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void embedding_kernel(const int64_t* __restrict__ ids,
                                                        const float* __restrict__ table, int D,
                                                        int vocab, float* __restrict__ out) {
  const int m = blockIdx.x;
  long id = ids[m];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // out-of-range ids are clamped, never read past the table
  const float4* src = reinterpret_cast<const float4*>(table + (size_t)id * D);
  float4* dst = reinterpret_cast<float4*>(out + (size_t)m * D);
  for (int i = threadIdx.x; i < D / 4; i += blockDim.x) dst[i] = src[i];
}

// ---------------------------------------------------------------------------------------------
// RMSNorm, optionally preceded by a residual add:
//   h_out = h (+ delta);  y = h_out * (w * 1/sqrt(mean(h_out^2) + eps))
// One workgroup per row. h_out may alias h; it is not written when delta is null.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ h,
                                                      const float* __restrict__ delta,
                                                      const float* __restrict__ w, int D, float eps,
                                                      float* h_out, float* __restrict__ y) {
  __shared__ float s_part[4];
  const size_t row = (size_t)blockIdx.x * D;
  float ss = 0.0f;
  for (int i = 4 * threadIdx.x; i < D; i += 4 * blockDim.x) {
    float4 v = *reinterpret_cast<const float4*>(h + row + i);
    if (delta) {
      const float4 d = *reinterpret_cast<const float4*>(delta + row + i);
      v.x += d.x;
      v.y += d.y;
      v.z += d.z;
      v.w += d.w;
      *reinterpret_cast<float4*>(h_out + row + i) = v;
    }
    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
  }
  const float mean = block_sum(ss, s_part) / (float)D;
  const float rstd = 1.0f / sqrtf(mean + eps);
  const float* src = delta ? h_out : h;  // this thread re-reads exactly what it wrote above
  for (int i = 4 * threadIdx.x; i < D; i += 4 * blockDim.x) {
    const float4 v = *reinterpret_cast<const float4*>(src + row + i);
    const float4 g = *reinterpret_cast<const float4*>(w + i);
    float4 o;
    o.x = v.x * (g.x * rstd);
    o.y = v.y * (g.y * rstd);
    o.z = v.z * (g.z * rstd);
    o.w = v.w * (g.w * rstd);
    *reinterpret_cast<float4*>(y + row + i) = o;
  }
}

// out = a + b, elementwise (n a multiple of 4)
__global__ __launch_bounds__(256) void add_kernel(const float* __restrict__ a,
                                                  const float* __restrict__ b, float* out, size_t n4) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n4) {
    const float4 x = reinterpret_cast<const float4*>(a)[i];
    const float4 y = reinterpret_cast<const float4*>(b)[i];
    reinterpret_cast<float4*>(out)[i] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
  }
}

// out = silu(g) * u = g / (1 + exp(-g)) * u
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ g,
                                                       const float* __restrict__ u,
                                                       float* __restrict__ out, size_t n4) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n4) {
    const float4 a = reinterpret_cast<const float4*>(g)[i];
    const float4 b = reinterpret_cast<const float4*>(u)[i];
    float4 o;
    o.x = silu_mul(a.x, b.x);
    o.y = silu_mul(a.y, b.y);
    o.z = silu_mul(a.z, b.z);
    o.w = silu_mul(a.w, b.w);
    reinterpret_cast<float4*>(out)[i] = o;
  }
}

// ---------------------------------------------------------------------------------------------
// RoPE tables: sin/cos [max_pos][D/2] (the reference stores each value twice, at d and d + D/2).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void rope_table_kernel(float* __restrict__ sin_t,
                                                        float* __restrict__ cos_t, int D, float base) {
  const int pos = blockIdx.x;
  const int half = D / 2;
  for (int d = threadIdx.x; d < half; d += blockDim.x) {
    float theta = 1.0f / powf(base, 2.0f * (float)d / (float)D);
    theta *= (float)pos;
    sin_t[(size_t)pos * half + d] = sinf(theta);
    cos_t[(size_t)pos * half + d] = cosf(theta);
  }
}

// ---------------------------------------------------------------------------------------------
// RoPE on q and k, then k and v into the cache at positions pos0 + m.
//   q [M][Hq*D] rotated in place; k, v [M][Hkv*D]; caches [Hkv][max_seq][D].
// grid (M, Hq + 2*Hkv), one wavefront per head vector. pos0 comes from device memory when
// d_pos0 is given (graph replay), else from the argument.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void rope_kv_kernel(float* __restrict__ q,
                                                     const float* __restrict__ k,
                                                     const float* __restrict__ v,
                                                     const float* __restrict__ sin_t,
                                                     const float* __restrict__ cos_t,
                                                     float* __restrict__ kc, float* __restrict__ vc,
                                                     int Hq, int Hkv, int D, int max_seq,
                                                     const int* __restrict__ d_pos0, int pos0) {
  const int m = blockIdx.x, head = blockIdx.y;
  const int half = D / 2;
  if (d_pos0) pos0 = *d_pos0;
  const int pos = pos0 + m;
  if (pos >= max_seq) return;  // the host checks capacity; a replayed graph past the end does nothing
  const float* st = sin_t + (size_t)pos * half;
  const float* ct = cos_t + (size_t)pos * half;
  if (head < Hq) {
    float* x = q + ((size_t)m * Hq + head) * D;
    for (int d = threadIdx.x; d < half; d += 64) {
      const float x0 = x[d], x1 = x[d + half], s = st[d], c = ct[d];
      x[d] = x0 * c - x1 * s;
      x[d + half] = x0 * s + x1 * c;
    }
  } else if (head < Hq + Hkv) {
    const int hk = head - Hq;
    const float* x = k + ((size_t)m * Hkv + hk) * D;
    float* dst = kc + ((size_t)hk * max_seq + pos) * D;
    for (int d = threadIdx.x; d < half; d += 64) {
      const float x0 = x[d], x1 = x[d + half], s = st[d], c = ct[d];
      dst[d] = x0 * c - x1 * s;
      dst[d + half] = x0 * s + x1 * c;
    }
  } else {
    const int hk = head - Hq - Hkv;
    const float* x = v + ((size_t)m * Hkv + hk) * D;
    float* dst = vc + ((size_t)hk * max_seq + pos) * D;
    for (int d = threadIdx.x; d < D; d += 64) dst[d] = x[d];
  }
}

// ---------------------------------------------------------------------------------------------
// Prefill attention: one query vector per wavefront over the cached keys 0..pos (head_dim 128).
//
// A wavefront takes 64 keys at a time: lane = key for the scores (each lane walks its key's row,
// q comes from LDS as a broadcast read), online softmax across chunks, then lane = 2 output
// dims for P*V (one coalesced 512-byte row per key, the weight broadcast with v_readlane).
// grid (Hq, M); query m sits at position pos0 + m.
// ---------------------------------------------------------------------------------------------
constexpr int kHeadDim = 128;
constexpr int kPartStride = kHeadDim + 2;

__global__ __launch_bounds__(64) void attention_prefill_kernel(const float* __restrict__ q,
                                                               const float* __restrict__ kc,
                                                               const float* __restrict__ vc,
                                                               float* __restrict__ out, int Hq, int Hkv,
                                                               int max_seq, const int* __restrict__ d_pos0,
                                                               int pos0, float scale, int key_stride,
                                                               int head_stride) {
  __shared__ __align__(16) float s_q[kHeadDim];
  const int h = blockIdx.x, lane = threadIdx.x;
  const int hk = h / (Hq / Hkv);
  if (d_pos0) pos0 = *d_pos0;
  const int m = blockIdx.y;
  const int end = min(pos0 + m + 1, max_seq);
  const float* qv = q + ((size_t)m * Hq + h) * kHeadDim;
  s_q[lane] = qv[lane];
  s_q[lane + 64] = qv[lane + 64];
  __syncthreads();

  // key `i` of KV head `hk` starts at hk * head_stride + i * key_stride floats: (128, max_seq * 128) for the
  // head-major cache of the decoder runner, (Hkv * 128, 128) for a [keys][Hkv][128] cache
  const float* kbase = kc + (size_t)hk * head_stride;
  const float* vbase = vc + (size_t)hk * head_stride;
  float run_max = -INFINITY, run_sum = 0.0f;
  float acc0 = 0.0f, acc1 = 0.0f;  // output dims 2*lane, 2*lane + 1

  for (int base = 0; base < end; base += 64) {
    const int key = base + lane;
    const bool valid = key < end;
    const float4* krow = reinterpret_cast<const float4*>(kbase + (size_t)(valid ? key : end - 1) * key_stride);
    float dot = 0.0f;
#pragma unroll 8
    for (int i = 0; i < kHeadDim / 4; ++i) {
      const float4 kv = krow[i];
      const float4 qq = *reinterpret_cast<const float4*>(s_q + 4 * i);
      dot += qq.x * kv.x;
      dot += qq.y * kv.y;
      dot += qq.z * kv.z;
      dot += qq.w * kv.w;
    }
    const float score = valid ? dot * scale : -INFINITY;
    const float new_max = fmaxf(run_max, wave_max(score));
    const float p = valid ? expf(score - new_max) : 0.0f;
    const float corr = expf(run_max - new_max);  // 0 on the first chunk (run_max = -inf)
    run_sum = run_sum * corr + wave_sum(p);
    acc0 *= corr;
    acc1 *= corr;
    run_max = new_max;
    const int cnt = min(64, end - base);
    for (int i0 = 0; i0 < cnt; i0 += 8) {
      // eight rows requested before the first is used (rows past cnt repeat the last, weight 0)
      float2 vv[8];
      float pi[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + u < cnt ? i0 + u : cnt - 1;
        vv[u] = *reinterpret_cast<const float2*>(vbase + (size_t)(base + i) * key_stride + 2 * lane);
        const float w = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), i));
        pi[u] = i0 + u < cnt ? w : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        acc0 += pi[u] * vv[u].x;
        acc1 += pi[u] * vv[u].y;
      }
    }
  }
  const float inv = 1.0f / run_sum;  // every query sees at least its own key
  float* o = out + ((size_t)m * Hq + h) * kHeadDim;
  *reinterpret_cast<float2*>(o + 2 * lane) = make_float2(acc0 * inv, acc1 * inv);
}

// ---------------------------------------------------------------------------------------------
// Prefill attention on the matrix cores, all in f32 (v_mfma_f32_32x32x2_f32): workgroup = one
// head x 32 queries, its 4 wavefronts take the 32-key blocks round-robin and are merged through LDS.
//
// Both products are computed transposed so that a lane always stands for one QUERY:
//   S^T = K Q^T   A = K block (lane: key l%32, dims 64*(l/32) + i), B = Q^T (lane: query l%32, same dims)
//                 C: lane = query l%32, register v = key 8*(v/4) + 4*(l/32) + v%4 of the block
//   O^T += V^T P^T  B = P^T = the softmaxed C registers as they are (step i uses register i: the
//                 two k-slots of the instruction are then keys 8*(i/4) + i%4 and that + 4),
//                 A = V^T (lane j = l%32 loads the float4 V[key][4j..4j+3]: component c feeds dim block c,
//                 whose row j stands for dim 4j + c)
//                 C: lane = query, register v of block c = dim 4*(8*(v/4) + 4*(l/32) + v%4) + c
// so the online-softmax statistics and the rescaling of O are per-lane scalars, and no operand
// needs a transpose.
// ---------------------------------------------------------------------------------------------
typedef float v16f32 __attribute__((ext_vector_type(16)));
// kPfWaves wavefronts per workgroup: 4, or 8 for long prompts (two wavefronts per SIMD overlap each
// other's loads and dependent MFMA chains; the merge area then takes 118 KB of LDS).
//
// kSplit: the key blocks of a query block are cut into up to kPfMaxChunks chunks of `cb` blocks, one
// workgroup each (blockIdx.z). A 32 x 32 block pair costs a SIMD 8192 clocks of f32 MFMA, and the last
// query block of a 512-token prompt has 16 of them: on one CU that alone is 33k clocks, while a fair share
// of the whole launch is 13k per SIMD. A query block with more than one chunk leaves (O, max, sum) per
// chunk in `part` and the last of its workgroups to finish combines them; with one chunk it writes the
// output directly.
constexpr int kPfMaxChunks = 8;
constexpr int kPfItemFloats = 66 * 64;       // one chunk's hand-over: 64 O^T registers, max, sum x 64 lanes

// Key blocks per chunk for a launch of M rows from position pos0 on: at least 4 (one per wavefront), at
// most kPfMaxChunks chunks per query block and about kPfTargetChunks in all (every chunk has a whole pass
// of loads, merge and hand-over to pay for, so more is not better).
constexpr int kPfTargetChunks = 768;
__device__ __forceinline__ int prefill_chunk_blocks(int pos0, int M, int max_seq, int Hq) {
  const int nqb = (M + 31) / 32;
  const int nkb_all = min(pos0 + M - 1, max_seq - 1) / 32 + 1;
  const int pairs = Hq * (nqb * (pos0 / 32) + nqb * (nqb + 1) / 2);  // (query block, key block) pairs
  const int by_total = (pairs + kPfTargetChunks - 1) / kPfTargetChunks;
  const int by_block = (nkb_all + kPfMaxChunks - 1) / kPfMaxChunks;
  const int cb = by_total > by_block ? by_total : by_block;
  return cb < 4 ? 4 : cb;
}

template <int kPfWaves, bool kSplit>
__global__ __launch_bounds__(64 * kPfWaves) void attention_prefill_mfma_kernel(
    const float* __restrict__ q, const float* __restrict__ kc, const float* __restrict__ vc,
    float* __restrict__ out, int M, int Hq, int Hkv, int max_seq, const int* __restrict__ d_pos0,
    int pos0, float scale, float* __restrict__ part, unsigned int* counters) {
  extern __shared__ __align__(16) float s_merge[];  // [kPfWaves - 1][66][64]: O^T registers, max, sum
  const int h = blockIdx.x, qb = blockIdx.y;
  const int hk = h / (Hq / Hkv);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int j = lane & 31, hh = lane >> 5;
  if (d_pos0) pos0 = *d_pos0;

  const int m_q = min(32 * qb + j, M - 1);           // this lane's query row (rows past M repeat the last)
  const int q_pos = pos0 + m_q;                        // its position: it sees keys 0..q_pos
  const int last_key = min(pos0 + min(32 * qb + 31, M - 1), max_seq - 1);
  const int nkb = last_key / 32 + 1;                   // key blocks this query block touches
  int kb_begin = 0, kb_end = nkb, nchunks = 1;
  if constexpr (kSplit) {
    const int cb = prefill_chunk_blocks(pos0, M, max_seq, Hq);
    nchunks = (nkb + cb - 1) / cb;
    kb_begin = (int)blockIdx.z * cb;
    kb_end = min(kb_begin + cb, nkb);
    if (kb_begin >= nkb) return;  // whole workgroup, before any barrier
  }

  float qreg[64];
  {
    const float4* src = reinterpret_cast<const float4*>(q + ((size_t)m_q * Hq + h) * kHeadDim + 64 * hh);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float4 v = src[i];
      qreg[4 * i] = v.x; qreg[4 * i + 1] = v.y; qreg[4 * i + 2] = v.z; qreg[4 * i + 3] = v.w;
    }
  }
  const float* kbase = kc + (size_t)hk * max_seq * kHeadDim;
  const float* vbase = vc + (size_t)hk * max_seq * kHeadDim;

  v16f32 o[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[c][v] = 0.0f;
  float run_max = -INFINITY, run_sum = 0.0f;

  for (int kb = kb_begin + wave; kb < kb_end; kb += kPfWaves) {
    // S^T block
    const int key_a = min(32 * kb + j, last_key);
    const float4* ksrc = reinterpret_cast<const float4*>(kbase + (size_t)key_a * kHeadDim + 64 * hh);
    v16f32 st;
#pragma unroll
    for (int v = 0; v < 16; ++v) st[v] = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float4 kv = ksrc[i];
      st = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qreg[4 * i], st, 0, 0, 0);
      st = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qreg[4 * i + 1], st, 0, 0, 0);
      st = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qreg[4 * i + 2], st, 0, 0, 0);
      st = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qreg[4 * i + 3], st, 0, 0, 0);
    }
    // V rows of this lane's 16 keys (both halves of the wavefront read whole 512-byte rows)
    float4 vreg[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int key = min(32 * kb + 8 * (v >> 2) + 4 * hh + (v & 3), last_key);
      vreg[v] = *reinterpret_cast<const float4*>(vbase + (size_t)key * kHeadDim + 4 * j);
    }
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
    // O^T += V^T P^T
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      o[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vreg[i].x, st[i], o[0], 0, 0, 0);
      o[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(vreg[i].y, st[i], o[1], 0, 0, 0);
      o[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(vreg[i].z, st[i], o[2], 0, 0, 0);
      o[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(vreg[i].w, st[i], o[3], 0, 0, 0);
    }
  }

  // wavefronts 1..3 hand their (max, sum, O^T) to wavefront 0
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
  float wmax[kPfWaves - 1], wsum[kPfWaves - 1];
  float total_max = run_max;
#pragma unroll
  for (int w = 0; w < kPfWaves - 1; ++w) {
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
  for (int w = 0; w < kPfWaves - 1; ++w) {
    const float wt = wmax[w] == -INFINITY ? 0.0f : __expf(wmax[w] - total_max);
    total_sum += wsum[w] * wt;
    const float* src = s_merge + (size_t)w * 66 * 64 + lane;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[c][v] += src[(16 * c + v) * 64] * wt;
  }
  // lane = query; register v of block c = dim 4*(8*(v/4) + 4*hh + v%4) + c: four blocks -> one float4
  if (kSplit && nchunks > 1) {
    // This chunk's (O^T registers, max, sum) go to scratch as [register][lane] (every store of the wavefront
    // is 256 contiguous bytes), written through to the device's coherence point; the last workgroup of the
    // query block to get here (arrival counter, left at 0) reads all chunks back and combines them.
    float* mine = part + (((size_t)h * gridDim.y + qb) * kPfMaxChunks) * kPfItemFloats + lane;
    float* dst = mine + (size_t)blockIdx.z * kPfItemFloats;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) store_shared_across_wgs(dst + (16 * c + v) * 64, o[c][v]);
    store_shared_across_wgs(dst + 64 * 64, total_max);
    store_shared_across_wgs(dst + 65 * 64, total_sum);
    stores_done();
    unsigned int* cnt = counters + (size_t)h * gridDim.y + qb;
    unsigned int prev = 0;
    if (lane == 0) prev = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = __shfl(prev, 0, 64);
    if (prev != (unsigned)nchunks - 1) return;
    arrivals_seen();
    float cmax[kPfMaxChunks], csum[kPfMaxChunks];
    float all_max = -INFINITY;
#pragma unroll
    for (int c = 0; c < kPfMaxChunks; ++c) {
      const float* ps = mine + (size_t)(c < nchunks ? c : 0) * kPfItemFloats;
      cmax[c] = load_shared_across_wgs(ps + 64 * 64);
      csum[c] = load_shared_across_wgs(ps + 65 * 64);
      if (c >= nchunks) cmax[c] = -INFINITY;
      all_max = fmaxf(all_max, cmax[c]);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[c][v] = 0.0f;
    total_sum = 0.0f;
    for (int ch = 0; ch < nchunks; ++ch) {
      const float wt = cmax[ch] == -INFINITY ? 0.0f : __expf(cmax[ch] - all_max);
      total_sum += csum[ch] * wt;
      const float* ps = mine + (size_t)ch * kPfItemFloats;
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[c][v] += load_shared_across_wgs(ps + (16 * c + v) * 64) * wt;
    }
    if (lane == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (32 * qb + j < M) {
    const float inv = 1.0f / total_sum;  // every query sees at least its own key
    float* dst = out + ((size_t)(32 * qb + j) * Hq + h) * kHeadDim;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = 8 * (v >> 2) + 4 * hh + (v & 3);
      *reinterpret_cast<float4*>(dst + 4 * row) =
          make_float4(o[0][v] * inv, o[1][v] * inv, o[2][v] * inv, o[3][v] * inv);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Decode attention (one query row): workgroup (x = group of kGW query heads that share a KV head,
// y = slice of the cached keys), 4 wavefronts per workgroup, each taking a quarter of the slice
// in blocks of 16 keys.
//
// Inside a wavefront 16 lanes share one key: lane (kq, dl) holds dims 8*dl..8*dl+7 of key slot kq,
// so a block's K and V rows are read as whole 512-byte rows, four rows per load instruction, and
// all of a block's loads are requested before the first is used. Scores are summed over the 16
// lanes with DPP adds, the softmax runs online per key slot, and the four slots, the four
// wavefronts (through LDS) and finally the workgroups of a head group (through `part`, by the last
// one to arrive) are merged with the usual max / rescale rule.
// ---------------------------------------------------------------------------------------------
constexpr int kDecWaves = 4;
constexpr int kMaxAttnSplit = 16;  // key slices per head group, at most

// d[g] += the same register of the other 15 lanes of the row (all lanes get the row's sum), for kGW
// independent values at once. A DPP operand must not be read within two wait states of the VALU write
// that produced it: the waits are part of the same asm statement as the instructions they protect (the
// compiler is free to schedule other instructions, the producer of d included, around a statement, but
// not into it), and with three values the other two adds of a step are the wait.
#define W4_DPP_ADD(n, ctrl) "v_add_f32_dpp %" #n ", %" #n ", %" #n " " ctrl " row_mask:0xf bank_mask:0xf\n\t"
#define W4_DPP_STEPS(ADDS, gap)                                                              \
  "s_nop 1\n\t" ADDS("quad_perm:[1,0,3,2]") gap ADDS("quad_perm:[2,3,0,1]") gap ADDS("row_half_mirror") gap \
      ADDS("row_mirror")
#define W4_DPP_ADDS1(ctrl) W4_DPP_ADD(0, ctrl)
#define W4_DPP_ADDS2(ctrl) W4_DPP_ADD(0, ctrl) W4_DPP_ADD(1, ctrl)
#define W4_DPP_ADDS3(ctrl) W4_DPP_ADD(0, ctrl) W4_DPP_ADD(1, ctrl) W4_DPP_ADD(2, ctrl)
template <int kGW>
__device__ __forceinline__ void row16_sum(float (&d)[kGW]) {
  static_assert(kGW >= 1 && kGW <= 3, "one to three values");
  if constexpr (kGW == 1) {
    asm volatile(W4_DPP_STEPS(W4_DPP_ADDS1, "s_nop 1\n\t") : "+v"(d[0]));
  } else if constexpr (kGW == 2) {
    asm volatile(W4_DPP_STEPS(W4_DPP_ADDS2, "s_nop 0\n\t") : "+v"(d[0]), "+v"(d[1]));
  } else {
    asm volatile(W4_DPP_STEPS(W4_DPP_ADDS3, "") : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]));
  }
}

// kRope: q, k_new, v_new are the raw outputs of the q/k/v Linears for the token at position pos0.
// The kernel rotates q itself, and the wavefront whose share contains key pos0 rotates k_new, uses
// it and v_new in place of the (not yet written) cache row and - in the first head group of each KV
// head - appends both to the cache. That is the RoPE + cache-append operator folded in.
// A lane holds dims 8*dl..8*dl+7; its RoPE partner dims (d +- 64) are read with a second load.
// kDefer: the workgroups of a head group do not meet. Each leaves its key slice's share where the Linear
// that reads the attention output (gemv_attn_rows_kernel) finds it and merges the slices while it loads
// its input row:  part[slice][head * 128 + d] = sum of exp(score - max) * v,  then, ns * Hq * 128 floats
// on,  [slice][head][2] = (max, sum of exp). That takes the hand-over (stores acknowledged, counter, reload)
// out of the chain of dependent memory round trips a decode step consists of.
template <int kGW, bool kRope, bool kDefer>
__global__ __launch_bounds__(64 * kDecWaves) void attention_decode_kernel(
    const int* __restrict__ d_pos0, const float* __restrict__ q, const float* __restrict__ sin_t,
    const float* __restrict__ cos_t, float* __restrict__ kc, float* __restrict__ vc, int Hq, int Hkv,
    int max_seq, int pos0,  // up to here the arguments arrive preloaded in SGPRs: what the first loads need
    int ns, float scale, const float* __restrict__ k_new, const float* __restrict__ v_new,
    float* __restrict__ out, float* part, unsigned int* counters) {
  __shared__ __align__(16) float s_part[4 * kDecWaves][kGW][kPartStride + 2];  // [wavefront x key slot]
  __shared__ unsigned int s_prev;
  const int h0 = blockIdx.x * kGW;             // first query head of this group
  const int G = Hq / Hkv;
  const int hk = h0 / G;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int kq = lane >> 4, dl = lane & 15;
  const int pdl = dl ^ 8;                      // the lane position that holds the RoPE partner dims
  if (d_pos0) pos0 = *d_pos0;                  // (a scalar load: nothing waits for it before its first use below)

  auto load8 = [](const float* src, float (&dst)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(src);
    const float4 b = *reinterpret_cast<const float4*>(src + 4);
    dst[0] = a.x; dst[1] = a.y; dst[2] = a.z; dst[3] = a.w;
    dst[4] = b.x; dst[5] = b.y; dst[6] = b.z; dst[7] = b.w;
  };
  // What does not depend on the position is requested while the position is on its way: q and (kRope) the new
  // token's k and v, each lane's own dims and, for the rotation, its partner's. Every wavefront asks for the
  // new k and v (three cached rows); only the one whose keys include the position uses them.
  float q_own[kGW][8], q_oth[kRope ? kGW : 1][8];
#pragma unroll
  for (int g = 0; g < kGW; ++g) {
    const float* src = q + (size_t)(h0 + g) * kHeadDim;
    load8(src + 8 * dl, q_own[g]);
    if (kRope) load8(src + 8 * pdl, q_oth[g]);
  }
  float kn_own[8], kn_oth[8], vnew[8];
  if (kRope) {
    load8(k_new + (size_t)hk * kHeadDim + 8 * dl, kn_own);
    load8(k_new + (size_t)hk * kHeadDim + 8 * pdl, kn_oth);
    load8(v_new + (size_t)hk * kHeadDim + 8 * dl, vnew);
  }
  __builtin_amdgcn_sched_barrier(0);

  if (pos0 >= max_seq) pos0 = max_seq - 1;     // the caller keeps the position inside the cache
  const int len = pos0 + 1;
  // keys of this workgroup, then of this wavefront (multiples of 4 so that slots stay aligned)
  const int per_wg = ((len + ns - 1) / ns + 15) / 16 * 16;
  const int per_wave = per_wg / kDecWaves;
  const int begin = min((int)blockIdx.y * per_wg + wave * per_wave, len);
  const int end = min(begin + per_wave, len);

  // y0 = x0 c - x1 s (first half of the head), y1 = x0 s + x1 c (second half)
  float sn[8], cs[8];
  if (kRope) {
    load8(sin_t + (size_t)pos0 * (kHeadDim / 2) + 8 * (dl & 7), sn);
    load8(cos_t + (size_t)pos0 * (kHeadDim / 2) + 8 * (dl & 7), cs);
  }
  auto rotate = [&](const float (&own)[8], const float (&oth)[8], float (&dst)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      dst[i] = dl < 8 ? own[i] * cs[i] - oth[i] * sn[i] : oth[i] * sn[i] + own[i] * cs[i];
    }
  };

  // The first block of K and V rows depends only on the position: it is requested as soon as that is known.
  const float* kbase = kc + (size_t)hk * max_seq * kHeadDim + 8 * dl;
  const float* vbase = vc + (size_t)hk * max_seq * kHeadDim + 8 * dl;
  float kk[4][8], vv[4][8];
  auto load_block = [&](int blk) {
    // all K rows before the V rows: loads return in issue order and the scores need K only
    const int last = end > begin ? end - 1 : 0;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int key = blk + 4 * it + kq;
      load8(kbase + (size_t)(key < end ? key : last) * kHeadDim, kk[it]);
    }
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int key = blk + 4 * it + kq;
      load8(vbase + (size_t)(key < end ? key : last) * kHeadDim, vv[it]);
    }
  };
  load_block(begin);

  float qr[kGW][8];
#pragma unroll
  for (int g = 0; g < kGW; ++g) {
    if (kRope) {
      rotate(q_own[g], q_oth[g], qr[g]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) qr[g][i] = q_own[g][i];
    }
  }
  float knew[8];
  const bool has_new = kRope && begin <= pos0 && pos0 < end;   // wavefront-uniform
  if (has_new) {
    rotate(kn_own, kn_oth, knew);
    if (h0 % G == 0 && blockIdx.x * kGW == (unsigned)h0 && kq == 0) {
      float* kd = kc + ((size_t)hk * max_seq + pos0) * kHeadDim + 8 * dl;
      float* vd = vc + ((size_t)hk * max_seq + pos0) * kHeadDim + 8 * dl;
      *reinterpret_cast<float4*>(kd) = make_float4(knew[0], knew[1], knew[2], knew[3]);
      *reinterpret_cast<float4*>(kd + 4) = make_float4(knew[4], knew[5], knew[6], knew[7]);
      *reinterpret_cast<float4*>(vd) = make_float4(vnew[0], vnew[1], vnew[2], vnew[3]);
      *reinterpret_cast<float4*>(vd + 4) = make_float4(vnew[4], vnew[5], vnew[6], vnew[7]);
    }
  }

  float m[kGW], l[kGW], acc[kGW][8];
#pragma unroll
  for (int g = 0; g < kGW; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.0f;
  }

  for (int blk = begin; blk < end; blk += 16) {
    if (blk != begin) load_block(blk);  // shares longer than 16 keys per wavefront (max_seq > 1024)
    if (has_new) {
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        // pos0 is this wavefront's last key: what lies behind it was loaded from the row of pos0 too
        // (clamped), which the cache does not hold yet. Those lanes get weight 0, but 0 x whatever
        // the memory held (Inf, NaN) must not reach the sums: they take the new row as well.
        const bool is_new = blk + 4 * it + kq >= pos0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          kk[it][i] = is_new ? knew[i] : kk[it][i];
          vv[it][i] = is_new ? vnew[i] : vv[it][i];
        }
      }
    }
    float sc[4][kGW];
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      float d[kGW];
#pragma unroll
      for (int g = 0; g < kGW; ++g) {
        float t = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) t += qr[g][i] * kk[it][i];
        d[g] = t;
      }
      row16_sum<kGW>(d);
      const bool valid = blk + 4 * it + kq < end;
#pragma unroll
      for (int g = 0; g < kGW; ++g) sc[it][g] = valid ? d[g] * scale : -INFINITY;
    }
#pragma unroll
    for (int g = 0; g < kGW; ++g) {
      const float bm = fmaxf(fmaxf(sc[0][g], sc[1][g]), fmaxf(sc[2][g], sc[3][g]));
      const float mn = fmaxf(m[g], bm);
      // mn stays -inf only while this slot has seen no valid key: everything it holds is 0
      const float corr = m[g] == -INFINITY ? 0.0f : __expf(m[g] - mn);
      l[g] *= corr;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[g][i] *= corr;
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const float p = sc[it][g] == -INFINITY ? 0.0f : __expf(sc[it][g] - mn);
        l[g] += p;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] += p * vv[it][i];
      }
      m[g] = mn;
    }
  }

  // Every key slot of every wavefront leaves its share in LDS; thread t (head t / 128, dim t % 128)
  // then merges the 16 of them. (Merging the four slots with cross-lane shuffles first cost three
  // times as long as these LDS reads.)
#pragma unroll
  for (int g = 0; g < kGW; ++g) {
    float* dst = &s_part[wave * 4 + kq][g][0];
    if (dl == 0) {
      dst[kHeadDim] = m[g];
      dst[kHeadDim + 1] = l[g];
    }
    *reinterpret_cast<float4*>(dst + 8 * dl) = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
    *reinterpret_cast<float4*>(dst + 8 * dl + 4) = make_float4(acc[g][4], acc[g][5], acc[g][6], acc[g][7]);
  }
  __syncthreads();

  for (int t = threadIdx.x; t < kGW * kHeadDim; t += 64 * kDecWaves) {
    const int g = t / kHeadDim, d = t % kHeadDim;
    float ms[4 * kDecWaves], ls[4 * kDecWaves], as[4 * kDecWaves];
#pragma unroll
    for (int w = 0; w < 4 * kDecWaves; ++w) {
      ms[w] = s_part[w][g][kHeadDim];
      ls[w] = s_part[w][g][kHeadDim + 1];
      as[w] = s_part[w][g][d];
    }
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4 * kDecWaves; ++w) mm = fmaxf(mm, ms[w]);
    float ll = 0.0f, a = 0.0f;
#pragma unroll
    for (int w = 0; w < 4 * kDecWaves; ++w) {
      const float wt = ms[w] == -INFINITY ? 0.0f : __expf(ms[w] - mm);
      ll += ls[w] * wt;
      a += as[w] * wt;
    }
    if (kDefer) {
      part[((size_t)blockIdx.y * Hq + h0 + g) * kHeadDim + d] = a;
      if (d == 0) {
        float* hdr = part + (size_t)ns * Hq * kHeadDim + ((size_t)blockIdx.y * Hq + h0 + g) * 2;
        *reinterpret_cast<float2*>(hdr) = make_float2(mm, ll);
      }
      continue;
    }
    float* mine = part + ((size_t)(h0 + g) * ns + blockIdx.y) * kPartStride;
    store_shared_across_wgs(mine + 2 + d, a);
    if (d == 0) {
      store_shared_across_wgs(mine, mm);
      store_shared_across_wgs(mine + 1, ll);
    }
  }
  if (kDefer) return;
  stores_done();
  __syncthreads();
  if (threadIdx.x == 0) {
    s_prev = __hip_atomic_fetch_add(counters + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (s_prev != (unsigned)ns - 1) return;
  arrivals_seen();
  // Last workgroup of this head group: merge the shares of all key slices. Every thread requests
  // all headers and its own dim of all shares at once (ns <= kMaxAttnSplit, loads independent).
  for (int t = threadIdx.x; t < kGW * kHeadDim; t += 64 * kDecWaves) {
    const int g = t / kHeadDim, d = t % kHeadDim;
    const float* all = part + (size_t)(h0 + g) * ns * kPartStride;
    float ms[kMaxAttnSplit], ls[kMaxAttnSplit], as[kMaxAttnSplit];
#pragma unroll
    for (int sidx = 0; sidx < kMaxAttnSplit; ++sidx) {
      const float* ps = all + (size_t)(sidx < ns ? sidx : ns - 1) * kPartStride;
      ms[sidx] = load_shared_across_wgs(ps);
      ls[sidx] = load_shared_across_wgs(ps + 1);
      as[sidx] = load_shared_across_wgs(ps + 2 + d);
    }
    float mm = -INFINITY;
#pragma unroll
    for (int sidx = 0; sidx < kMaxAttnSplit; ++sidx) mm = fmaxf(mm, sidx < ns ? ms[sidx] : -INFINITY);
    float ll = 0.0f, a = 0.0f;
#pragma unroll
    for (int sidx = 0; sidx < kMaxAttnSplit; ++sidx) {
      const float wt = (sidx < ns && ms[sidx] != -INFINITY) ? __expf(ms[sidx] - mm) : 0.0f;
      ll += ls[sidx] * wt;
      a += as[sidx] * wt;
    }
    out[(size_t)(h0 + g) * kHeadDim + d] = a / ll;  // key 0 is always there: ll > 0
  }
  if (threadIdx.x == 0) {  // ready for the next launch
    __hip_atomic_store(counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// ---------------------------------------------------------------------------------------------
// Greedy argmax over one row of logits: the first maximum wins. Workgroups reduce slices, the
// last one to finish (arrival counter) reduces the per-workgroup results, writes the token and,
// when given, advances the position counter of the decoder state.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void argmax_merge(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i < bi)) {
    bv = v;
    bi = i;
  }
}

__global__ __launch_bounds__(256) void argmax_kernel(const float* __restrict__ logits, int n,
                                                     float* part_val, int* part_idx,
                                                     unsigned int* counter, int64_t* __restrict__ token_out,
                                                     int* pos_to_advance) {
  __shared__ float s_val[256];
  __shared__ int s_idx[256];
  __shared__ unsigned int s_prev;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
    argmax_merge(bv, bi, logits[i], i);
  }
  s_val[threadIdx.x] = bv;
  s_idx[threadIdx.x] = bi;
  __syncthreads();
  for (int off = 128; off >= 1; off >>= 1) {
    if ((int)threadIdx.x < off) {
      float v = s_val[threadIdx.x];
      int i = s_idx[threadIdx.x];
      argmax_merge(v, i, s_val[threadIdx.x + off], s_idx[threadIdx.x + off]);
      s_val[threadIdx.x] = v;
      s_idx[threadIdx.x] = i;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    store_shared_across_wgs(part_val + blockIdx.x, s_val[0]);
    store_shared_across_wgs(part_idx + blockIdx.x, s_idx[0]);
    stores_done();
    s_prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (s_prev != gridDim.x - 1) return;
  arrivals_seen();
  bv = -INFINITY;
  bi = 0x7fffffff;
  for (int b = threadIdx.x; b < (int)gridDim.x; b += blockDim.x) {
    argmax_merge(bv, bi, load_shared_across_wgs(part_val + b), load_shared_across_wgs(part_idx + b));
  }
  s_val[threadIdx.x] = bv;
  s_idx[threadIdx.x] = bi;
  __syncthreads();
  for (int off = 128; off >= 1; off >>= 1) {
    if ((int)threadIdx.x < off) {
      float v = s_val[threadIdx.x];
      int i = s_idx[threadIdx.x];
      argmax_merge(v, i, s_val[threadIdx.x + off], s_idx[threadIdx.x + off]);
      s_val[threadIdx.x] = v;
      s_idx[threadIdx.x] = i;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const int best = s_idx[0] == 0x7fffffff ? 0 : s_idx[0];  // all -inf / NaN: token 0, as the reference's scan
    *token_out = best;
    __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (pos_to_advance) *pos_to_advance += 1;
  }
}

// The same decision from partial results: (value, index) pairs, each the first maximum of a disjoint set of
// logits, as the lm_head launch leaves them (one pair per wavefront; n <= 4096). One workgroup of 1024 threads:
// every thread requests its four pairs at once, wavefronts reduce with shuffles, the first one finishes.
__global__ __launch_bounds__(1024) void argmax_parts_kernel(const float* __restrict__ val,
                                                            const int* __restrict__ idx, int n,
                                                            int64_t* __restrict__ token_out, int* pos_to_advance) {
  __shared__ float s_val[16];
  __shared__ int s_idx[16];
  float v[4];
  int ix[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int i = (int)threadIdx.x + 1024 * k;
    const int ic = i < n ? i : n - 1;  // a duplicate of a real pair: harmless
    v[k] = val[ic];
    ix[k] = idx[ic];
  }
  float bv = v[0];
  int bi = ix[0];
#pragma unroll
  for (int k = 1; k < 4; ++k) argmax_merge(bv, bi, v[k], ix[k]);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float ov = __shfl_xor(bv, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    argmax_merge(bv, bi, ov, oi);
  }
  if ((threadIdx.x & 63) == 0) {
    s_val[threadIdx.x >> 6] = bv;
    s_idx[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    bv = s_val[threadIdx.x & 15];
    bi = s_idx[threadIdx.x & 15];
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      argmax_merge(bv, bi, ov, oi);
    }
    if (threadIdx.x == 0) {
      *token_out = bi == 0x7fffffff ? 0 : bi;  // all -inf / NaN: token 0, as the reference's scan
      if (pos_to_advance) *pos_to_advance += 1;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// im2col for a Conv3D without padding and dilation (the vision patch embedding), so that the
// convolution becomes the same quantized Linear: row = (b, ot, oh, ow), column = (c, kt, kh, kw),
// as im2col_conv3d_p0_d1_activation_fp32 (mllm/Backends/Arm/Kernels/conv3d.cpp:15-78) lays it out.
// Columns from the true width up to ld are written as 0 (K is padded to a multiple of 32 for the
// block-32 weights; a zero column changes neither the row's quantisation range nor any sum).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void im2col_conv3d_kernel(const float* __restrict__ a,
                                                            float* __restrict__ z, int C, int T, int H,
                                                            int W, int kt, int kh, int kw, int st, int sh,
                                                            int sw, int OT, int OH, int OW, int ld) {
  const int row = blockIdx.x;  // (b, ot, oh, ow)
  const int ow = row % OW, oh = (row / OW) % OH, ot = (row / (OW * OH)) % OT, b = row / (OW * OH * OT);
  const int kvol = kt * kh * kw, cols = C * kvol;
  const float* ab = a + (size_t)b * C * T * H * W;
  float* zr = z + (size_t)row * ld;
  for (int col = threadIdx.x; col < ld; col += blockDim.x) {
    float v = 0.0f;
    if (col < cols) {
      const int c = col / kvol, r = col % kvol;
      const int dt = r / (kh * kw), dh = (r / kw) % kh, dw = r % kw;
      v = ab[(((size_t)c * T + (ot * st + dt)) * H + (oh * sh + dh)) * W + (ow * sw + dw)];
    }
    zr[col] = v;
  }
}

__global__ void add_to_int_kernel(int* p, int delta) { *p += delta; }
__global__ void set_int_kernel(int* p, int value) { *p = value; }
__global__ void zero_u32_kernel(unsigned int* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// ---------------------------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------------------------
hipError_t launch_embedding(const int64_t* ids, const float* table, int M, int D, int vocab,
                            float* out, hipStream_t s) {
  hipLaunchKernelGGL(embedding_kernel, dim3(M), dim3(256), 0, s, ids, table, D, vocab, out);
  return hipGetLastError();
}

hipError_t launch_rmsnorm(const float* h, const float* delta, const float* w, int M, int D, float eps,
                          float* h_out, float* y, hipStream_t s) {
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(M), dim3(256), 0, s, h, delta, w, D, eps, h_out, y);
  return hipGetLastError();
}

hipError_t launch_add(const float* a, const float* b, float* out, size_t n, hipStream_t s) {
  const size_t n4 = n / 4;
  hipLaunchKernelGGL(add_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, a, b, out, n4);
  return hipGetLastError();
}

hipError_t launch_silu_mul(const float* g, const float* u, float* out, size_t n, hipStream_t s) {
  const size_t n4 = n / 4;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, g, u, out, n4);
  return hipGetLastError();
}

hipError_t launch_rope_table(float* sin_t, float* cos_t, int max_pos, int D, float base, hipStream_t s) {
  hipLaunchKernelGGL(rope_table_kernel, dim3(max_pos), dim3(64), 0, s, sin_t, cos_t, D, base);
  return hipGetLastError();
}

hipError_t launch_rope_kv(float* q, const float* k, const float* v, const float* sin_t,
                          const float* cos_t, float* kc, float* vc, int M, int Hq, int Hkv, int D,
                          int max_seq, const int* d_pos0, int pos0, hipStream_t s) {
  hipLaunchKernelGGL(rope_kv_kernel, dim3(M, Hq + 2 * Hkv), dim3(64), 0, s, q, k, v, sin_t, cos_t, kc,
                     vc, Hq, Hkv, D, max_seq, d_pos0, pos0);
  return hipGetLastError();
}

// Scratch of the chunked launch: arrival counters (one per head and query block, 256-byte aligned) in front
// of the chunks' hand-over areas.
static size_t pf_counter_bytes(int M, int Hq) {
  return (sizeof(unsigned int) * (size_t)Hq * ((M + 31) / 32) + 255) / 256 * 256;
}
size_t attention_prefill_part_bytes(int M, int Hq) {
  return pf_counter_bytes(M, Hq) +
         sizeof(float) * (size_t)Hq * ((M + 31) / 32) * kPfMaxChunks * kPfItemFloats;
}

// part: optional scratch of attention_prefill_part_bytes(M, Hq) bytes; with it, and when the query blocks
// alone would leave half of the CUs idle, the key range of a query block is dealt to several workgroups
// and the last of them to finish combines their results.
// counters: optional Hq * ceil(M / 32) words that are 0 and are left 0; without them the head of `part`
// serves and is cleared by a launch of its own first.
// Measured (12 heads; unsplit -> chunked, counters given): 256 rows at position 0: 19 -> 16 us, at 768:
// 46 -> 40; 128 rows at 3000: 218 -> 64; 64 at 2000: 134 -> 39; 32 at 500: 38 -> 17. From 384 rows on the
// unsplit kernel's 8 wavefronts with several key blocks each do better when the prompt continues a long
// context (512 rows at 512: 49 against 63 us), so those sizes stay unsplit (512 rows at 0: 29.4 against 26).
hipError_t launch_attention_prefill(const float* q, const float* kc, const float* vc, float* out,
                                    int M, int Hq, int Hkv, int max_seq, const int* d_pos0, int pos0,
                                    float* part, size_t part_bytes, unsigned int* counters, hipStream_t s) {
  const float scale = 1.0f / sqrtf((float)kHeadDim);
  if (M >= 16 && Hq * ((M + 31) / 32) <= 128 && part && part_bytes >= attention_prefill_part_bytes(M, Hq)) {
    constexpr int W = 4;
    const size_t lds = sizeof(float) * (W - 1) * 66 * 64;
    const dim3 grid(Hq, (M + 31) / 32, kPfMaxChunks);
    if (!counters) {
      counters = reinterpret_cast<unsigned int*>(part);
      if (hipError_t e = launch_zero_u32(counters, Hq * ((M + 31) / 32), s); e != hipSuccess) return e;
    }
    float* areas = part + pf_counter_bytes(M, Hq) / sizeof(float);
    hipLaunchKernelGGL((attention_prefill_mfma_kernel<W, true>), grid, dim3(64 * W), lds, s, q, kc, vc, out,
                       M, Hq, Hkv, max_seq, d_pos0, pos0, scale, areas, counters);
    return hipGetLastError();
  }
  if (M >= 256) {  // matrix-core kernel, 32 queries per workgroup; many key blocks: 8 wavefronts
    constexpr int W = 8;
    const size_t lds = sizeof(float) * (W - 1) * 66 * 64;
    static LdsLimitOnce raised;  // 118 KB of dynamic LDS: above the default limit
    if (hipError_t e = raised.raise(reinterpret_cast<const void*>(attention_prefill_mfma_kernel<W, false>), lds);
        e != hipSuccess)
      return e;
    hipLaunchKernelGGL((attention_prefill_mfma_kernel<W, false>), dim3(Hq, (M + 31) / 32), dim3(64 * W), lds,
                       s, q, kc, vc, out, M, Hq, Hkv, max_seq, d_pos0, pos0, scale, nullptr, nullptr);
  } else if (M >= 16) {
    constexpr int W = 4;
    const size_t lds = sizeof(float) * (W - 1) * 66 * 64;
    hipLaunchKernelGGL((attention_prefill_mfma_kernel<W, false>), dim3(Hq, (M + 31) / 32), dim3(64 * W), lds,
                       s, q, kc, vc, out, M, Hq, Hkv, max_seq, d_pos0, pos0, scale, nullptr, nullptr);
  } else {
    hipLaunchKernelGGL(attention_prefill_kernel, dim3(Hq, M), dim3(64), 0, s, q, kc, vc, out, Hq, Hkv,
                       max_seq, d_pos0, pos0, scale, kHeadDim, max_seq * kHeadDim);
  }
  return hipGetLastError();
}

// The one-wavefront-per-query kernel on K / V laid out [keys][Hkv][128] (the reference's kBSHD_NO_REPEAT
// cache at batch 1): what the engine's FlashAttn2 operator is handed.
hipError_t launch_attention_bshd(const float* q, const float* k, const float* v, float* out, int M, int Hq,
                                 int Hkv, int n_keys, int pos0, hipStream_t s) {
  const float scale = 1.0f / sqrtf((float)kHeadDim);
  hipLaunchKernelGGL(attention_prefill_kernel, dim3(Hq, M), dim3(64), 0, s, q, k, v, out, Hq, Hkv, n_keys,
                     nullptr, pos0, scale, Hkv * kHeadDim, kHeadDim);
  return hipGetLastError();
}

// k_new != null: q, k_new, v_new are un-rotated Linear outputs of the token at pos0 and the kernel
// performs RoPE and the cache append itself (then sin_t / cos_t are the RoPE tables).
hipError_t launch_attention_decode(const float* q, float* kc, float* vc, float* out, int Hq, int Hkv,
                                   int max_seq, const int* d_pos0, int pos0, int nsplit, float* part,
                                   unsigned int* counters, const float* k_new, const float* v_new,
                                   const float* sin_t, const float* cos_t, bool defer, hipStream_t s) {
  const float scale = 1.0f / sqrtf((float)kHeadDim);
  const int G = Hq / Hkv;  // query heads per KV head; a workgroup takes 2 or 3 of them when it divides
  if (nsplit > kMaxAttnSplit) return hipErrorInvalidValue;
#define W4_ATTN_D(gw, rope, df)                                                                            \
  hipLaunchKernelGGL((attention_decode_kernel<gw, rope, df>), dim3(Hq / gw, nsplit), dim3(64 * kDecWaves), \
                     0, s, d_pos0, q, sin_t, cos_t, kc, vc, Hq, Hkv, max_seq, pos0, nsplit, scale,         \
                     k_new, v_new, out, part, counters)
#define W4_ATTN(gw, rope) W4_ATTN_D(gw, rope, false)
  if (defer) {  // the slices are left for the Linear that follows: the folded RoPE form only
    if (!k_new) return hipErrorInvalidValue;
    if (G % 2 == 0) W4_ATTN_D(2, true, true);
    else if (G % 3 == 0) W4_ATTN_D(3, true, true);
    else W4_ATTN_D(1, true, true);
    return hipGetLastError();
  }
  if (G % 2 == 0) {
    if (k_new) W4_ATTN(2, true); else W4_ATTN(2, false);
  } else if (G % 3 == 0) {
    if (k_new) W4_ATTN(3, true); else W4_ATTN(3, false);
  } else {
    if (k_new) W4_ATTN(1, true); else W4_ATTN(1, false);
  }
#undef W4_ATTN
#undef W4_ATTN_D
  return hipGetLastError();
}

hipError_t launch_argmax(const float* logits, int n, float* part_val, int* part_idx,
                         unsigned int* counter, int64_t* token_out, int* pos_to_advance, int blocks,
                         hipStream_t s) {
  hipLaunchKernelGGL(argmax_kernel, dim3(blocks), dim3(256), 0, s, logits, n, part_val, part_idx,
                     counter, token_out, pos_to_advance);
  return hipGetLastError();
}

hipError_t launch_argmax_parts(const float* val, const int* idx, int n, int64_t* token_out, int* pos_to_advance,
                               hipStream_t s) {
  if (n <= 0 || n > 4096) return hipErrorInvalidValue;
  hipLaunchKernelGGL(argmax_parts_kernel, dim3(1), dim3(1024), 0, s, val, idx, n, token_out, pos_to_advance);
  return hipGetLastError();
}

hipError_t launch_im2col_conv3d(const float* a, float* z, int B, int C, int T, int H, int W, int kt,
                                int kh, int kw, int st, int sh, int sw, int ld, hipStream_t s) {
  const int OT = (T - kt) / st + 1, OH = (H - kh) / sh + 1, OW = (W - kw) / sw + 1;
  hipLaunchKernelGGL(im2col_conv3d_kernel, dim3(B * OT * OH * OW), dim3(256), 0, s, a, z, C, T, H, W, kt,
                     kh, kw, st, sh, sw, OT, OH, OW, ld);
  return hipGetLastError();
}

hipError_t launch_set_int(int* p, int value, hipStream_t s) {
  hipLaunchKernelGGL(set_int_kernel, dim3(1), dim3(1), 0, s, p, value);
  return hipGetLastError();
}

hipError_t launch_add_to_int(int* p, int delta, hipStream_t s) {
  hipLaunchKernelGGL(add_to_int_kernel, dim3(1), dim3(1), 0, s, p, delta);
  return hipGetLastError();
}

hipError_t launch_zero_u32(unsigned int* p, int n, hipStream_t s) {
  hipLaunchKernelGGL(zero_u32_kernel, dim3((n + 255) / 256), dim3(256), 0, s, p, n);
  return hipGetLastError();
}

}  // namespace w4
