// Operators that only the engine's op-by-op path needs (the decoder runner fuses them away): SiLU and
// element-wise multiply on their own, RoPE on one tensor, and a dense f32 matmul against a row-major
// [N][K] operand (the reference multiplies by its lm_head that way). f32 throughout.
//
// Reference behaviour followed (file:line in the reference tree):
//   SiLU        mllm/Backends/Arm/Ops/SiLUOp.cpp               y = x / (1 + exp(-x))
//   Mul         mllm/Backends/Arm/Ops/ElewiseOps.cpp           same-shape element-wise product
//   RoPE        mllm/Backends/Arm/Kernels/rope.cpp:39-80       half-split pairs, rows [S][H][D] (layout kBSHD)
//   MatMul      mllm/Backends/Arm/Ops/MatMulOp.cpp:131-167     C = A B^T (transpose_b), f32
#include "w4a32_decoder.h"
#include "w4a32_internal.h"

namespace w4 {

namespace {

// silu(g) = g * rcp(1 + exp2(-g * log2 e)): silu_mul()'s first factor, so that SiLU followed by Mul gives
// what the fused operator gives, bit for bit
__device__ __forceinline__ float silu_one(float g) {
  const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
  return g * __builtin_amdgcn_rcpf(1.0f + e);
}

__global__ __launch_bounds__(256) void silu_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                   size_t n4) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n4) {
    const float4 a = reinterpret_cast<const float4*>(x)[i];
    reinterpret_cast<float4*>(out)[i] = make_float4(silu_one(a.x), silu_one(a.y), silu_one(a.z), silu_one(a.w));
  }
}

__global__ __launch_bounds__(256) void mul_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                  float* out, size_t n4) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n4) {
    const float4 x = reinterpret_cast<const float4*>(a)[i];
    const float4 y = reinterpret_cast<const float4*>(b)[i];
    reinterpret_cast<float4*>(out)[i] = make_float4(x.x * y.x, x.y * y.y, x.z * y.z, x.w * y.w);
  }
}

// y[m][h][:] = rope(x[m][h][:]) at position pos0 + m; grid (M, H), one wavefront per head vector.
// The arithmetic of rope_kv_kernel (y0 = x0 c - x1 s, y1 = x0 s + x1 c, unfused products).
__global__ __launch_bounds__(64) void rope_rows_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                       const float* __restrict__ sin_t,
                                                       const float* __restrict__ cos_t, int H, int D, int pos0) {
  const int m = blockIdx.x, head = blockIdx.y, half = D / 2;
  const float* st = sin_t + (size_t)(pos0 + m) * half;
  const float* ct = cos_t + (size_t)(pos0 + m) * half;
  const float* src = x + ((size_t)m * H + head) * D;
  float* dst = y + ((size_t)m * H + head) * D;
  for (int d = threadIdx.x; d < half; d += 64) {
    const float x0 = src[d], x1 = src[d + half], s = st[d], c = ct[d];
    dst[d] = x0 * c - x1 * s;
    dst[d + half] = x0 * s + x1 * c;
  }
}

__device__ __forceinline__ float wave_total(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// C[m][n] = sum_k A[m][k] B[n][k] for M <= 8 rows: a stream over B, which is read once. A wavefront
// owns kRows consecutive rows of B and walks K in steps of 256 floats (one float4 per lane and row);
// A's rows come from the cache. HBM-bound: N * K * 4 bytes.
constexpr int kGemvRows = 4;
template <int M>
__global__ __launch_bounds__(256) void dense_gemv_kernel(const float* __restrict__ a,
                                                         const float* __restrict__ b, float* __restrict__ c,
                                                         int N, int K) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n0 = ((int)blockIdx.x * 4 + wave) * kGemvRows;
  if (n0 >= N) return;
  float acc[M][kGemvRows];
#pragma unroll
  for (int m = 0; m < M; ++m)
#pragma unroll
    for (int r = 0; r < kGemvRows; ++r) acc[m][r] = 0.0f;
  const float* brow[kGemvRows];
#pragma unroll
  for (int r = 0; r < kGemvRows; ++r) brow[r] = b + (size_t)(n0 + r < N ? n0 + r : N - 1) * K;
#pragma unroll 2
  for (int k = 4 * lane; k < K; k += 256) {
    float4 bv[kGemvRows];
#pragma unroll
    for (int r = 0; r < kGemvRows; ++r) bv[r] = *reinterpret_cast<const float4*>(brow[r] + k);
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float4 av = *reinterpret_cast<const float4*>(a + (size_t)m * K + k);
#pragma unroll
      for (int r = 0; r < kGemvRows; ++r) {
        acc[m][r] += av.x * bv[r].x;
        acc[m][r] += av.y * bv[r].y;
        acc[m][r] += av.z * bv[r].z;
        acc[m][r] += av.w * bv[r].w;
      }
    }
  }
#pragma unroll
  for (int m = 0; m < M; ++m)
#pragma unroll
    for (int r = 0; r < kGemvRows; ++r) {
      const float t = wave_total(acc[m][r]);
      if (lane == 0 && n0 + r < N) c[(size_t)m * N + n0 + r] = t;
    }
}

// The same product for more rows on the matrix cores in f32 (v_mfma_f32_32x32x2_f32): a workgroup of four
// wavefronts owns a 64 x 64 tile of C, each wavefront a 32 x 32 quarter; A and B tiles of 16 k go through
// LDS ([row][16 + 1] floats, the pad keeps the operand reads off one bank). A plain kernel for an operator
// the decoder runner does not use: every row's logits of a prompt are computed, as the reference does.
// B may be held as f16 (BT = _Float16): its elements widen to f32 exactly on the way into LDS.
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
constexpr int kMmTile = 64, kMmK = 16, kMmLd = kMmK + 1;
__device__ __forceinline__ float4 load4_as_f32(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4_as_f32(const _Float16* p) {
  const h4_t h = *reinterpret_cast<const h4_t*>(p);
  return make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
}
template <typename BT>
__global__ __launch_bounds__(256) void dense_gemm_kernel(const float* __restrict__ a, const BT* __restrict__ b,
                                                         float* __restrict__ c, int M, int N, int K) {
  __shared__ float s_a[kMmTile * kMmLd], s_b[kMmTile * kMmLd];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int m0 = blockIdx.y * kMmTile, n0 = blockIdx.x * kMmTile;
  const int wm = 32 * (wave >> 1), wn = 32 * (wave & 1);
  // loader: thread t brings A[m0 + t/4][k0 + 4*(t%4) ..+3] and the same of B (K % 4 == 0)
  const int lr = threadIdx.x >> 2, lk = 4 * (threadIdx.x & 3);
  const float* ap = a + (size_t)(m0 + lr < M ? m0 + lr : M - 1) * K + lk;
  const BT* bp = b + (size_t)(n0 + lr < N ? n0 + lr : N - 1) * K + lk;
  v16f acc = {0};
  for (int k0 = 0; k0 < K; k0 += kMmK) {
    float4 av = make_float4(0, 0, 0, 0), bv = make_float4(0, 0, 0, 0);
    if (k0 + lk < K) {
      av = *reinterpret_cast<const float4*>(ap + k0);
      bv = load4_as_f32(bp + k0);
    }
    __syncthreads();  // the previous step's reads are done
    s_a[lr * kMmLd + lk + 0] = av.x; s_a[lr * kMmLd + lk + 1] = av.y;
    s_a[lr * kMmLd + lk + 2] = av.z; s_a[lr * kMmLd + lk + 3] = av.w;
    s_b[lr * kMmLd + lk + 0] = bv.x; s_b[lr * kMmLd + lk + 1] = bv.y;
    s_b[lr * kMmLd + lk + 2] = bv.z; s_b[lr * kMmLd + lk + 3] = bv.w;
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kMmK; kk += 2) {
      // A operand: lane = row lane % 32, k = kk + lane / 32; B operand: lane = column lane % 32, same k
      const float af = s_a[(wm + (lane & 31)) * kMmLd + kk + (lane >> 5)];
      const float bf = s_b[(wn + (lane & 31)) * kMmLd + kk + (lane >> 5)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af, bf, acc, 0, 0, 0);
    }
  }
  // C layout of the 32 x 32 accumulator: column lane % 32, row 8 * (v / 4) + 4 * (lane / 32) + v % 4
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = m0 + wm + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
    const int col = n0 + wn + (lane & 31);
    if (row < M && col < N) c[(size_t)row * N + col] = acc[v];
  }
}

}  // namespace

hipError_t launch_silu(const float* x, float* out, size_t n, hipStream_t s) {
  const size_t n4 = n / 4;
  hipLaunchKernelGGL(silu_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, x, out, n4);
  return hipGetLastError();
}

hipError_t launch_mul(const float* a, const float* b, float* out, size_t n, hipStream_t s) {
  const size_t n4 = n / 4;
  hipLaunchKernelGGL(mul_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, a, b, out, n4);
  return hipGetLastError();
}

hipError_t launch_rope_rows(const float* x, float* y, const float* sin_t, const float* cos_t, int M, int H,
                            int D, int pos0, hipStream_t s) {
  hipLaunchKernelGGL(rope_rows_kernel, dim3(M, H), dim3(64), 0, s, x, y, sin_t, cos_t, H, D, pos0);
  return hipGetLastError();
}

hipError_t launch_matmul_nt(const float* a, const void* b, int b_dtype, float* c, int M, int N, int K,
                            hipStream_t s) {
  // few rows: a stream over B (f16 or f32), 16 lanes per row of B
  if (dense_rows_applies(M, K)) return launch_dense_rows(a, K, b, b_dtype, c, M, N, K, s);
  const dim3 tiles((N + kMmTile - 1) / kMmTile, (M + kMmTile - 1) / kMmTile);
  if (b_dtype == W4A32_DENSE_F16) {
    hipLaunchKernelGGL(dense_gemm_kernel<_Float16>, tiles, dim3(256), 0, s, a, static_cast<const _Float16*>(b), c, M,
                       N, K);
    return hipGetLastError();
  }
  if (b_dtype != W4A32_DENSE_F32) return hipErrorInvalidValue;
  return launch_matmul_f32_nt(a, static_cast<const float*>(b), c, M, N, K, s);
}

hipError_t launch_matmul_f32_nt(const float* a, const float* b, float* c, int M, int N, int K, hipStream_t s) {
  if (dense_rows_applies(M, K)) return launch_dense_rows(a, K, b, W4A32_DENSE_F32, c, M, N, K, s);
  if (M <= 8) {
    const dim3 grid((N + 4 * kGemvRows - 1) / (4 * kGemvRows));
#define W4_DENSE_GEMV(MM) \
  case MM: hipLaunchKernelGGL(dense_gemv_kernel<MM>, grid, dim3(256), 0, s, a, b, c, N, K); break
    switch (M) {
      W4_DENSE_GEMV(1); W4_DENSE_GEMV(2); W4_DENSE_GEMV(3); W4_DENSE_GEMV(4);
      W4_DENSE_GEMV(5); W4_DENSE_GEMV(6); W4_DENSE_GEMV(7); W4_DENSE_GEMV(8);
    }
#undef W4_DENSE_GEMV
    return hipGetLastError();
  }
  hipLaunchKernelGGL(dense_gemm_kernel<float>, dim3((N + kMmTile - 1) / kMmTile, (M + kMmTile - 1) / kMmTile),
                     dim3(256), 0, s, a, b, c, M, N, K);
  return hipGetLastError();
}

}  // namespace w4

namespace {
inline int from_hip(hipError_t e) { return e == hipSuccess ? W4A32_OK : W4A32_ELAUNCH; }
inline hipStream_t S(void* stream) { return static_cast<hipStream_t>(stream); }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
}  // namespace

extern "C" {

int w4a32_op_silu(const float* d_x, float* d_out, size_t n, void* stream) {
  if (!d_x || !d_out || n == 0) return W4A32_EINVAL;
  if (n % 4 != 0) return W4A32_ESHAPE;
  return from_hip(w4::launch_silu(d_x, d_out, n, S(stream)));
}

int w4a32_op_mul(const float* d_a, const float* d_b, float* d_out, size_t n, void* stream) {
  if (!d_a || !d_b || !d_out || n == 0) return W4A32_EINVAL;
  if (n % 4 != 0) return W4A32_ESHAPE;
  return from_hip(w4::launch_mul(d_a, d_b, d_out, n, S(stream)));
}

int w4a32_op_rope(const float* d_x, float* d_y, const float* d_sin, const float* d_cos, int M, int n_heads,
                  int head_dim, int pos0, int table_rows, void* stream) {
  if (!d_x || !d_y || !d_sin || !d_cos) return W4A32_EINVAL;
  if (M <= 0 || n_heads <= 0 || head_dim <= 0 || pos0 < 0) return W4A32_EINVAL;
  if (head_dim % 2 != 0 || pos0 + M > table_rows) return W4A32_ESHAPE;
  return from_hip(w4::launch_rope_rows(d_x, d_y, d_sin, d_cos, M, n_heads, head_dim, pos0, S(stream)));
}

int w4a32_op_attention_bshd(const float* d_q, const float* d_k, const float* d_v, float* d_out, int M,
                            int n_heads, int n_kv_heads, int head_dim, int n_keys, int pos0, void* stream) {
  if (!d_q || !d_k || !d_v || !d_out) return W4A32_EINVAL;
  if (M <= 0 || n_heads <= 0 || n_kv_heads <= 0 || n_keys <= 0 || pos0 < 0) return W4A32_EINVAL;
  if (head_dim != 128 || n_heads % n_kv_heads != 0 || pos0 + M > n_keys) return W4A32_ESHAPE;
  if (!aligned16(d_q) || !aligned16(d_k) || !aligned16(d_v) || !aligned16(d_out)) return W4A32_EINVAL;
  return from_hip(w4::launch_attention_bshd(d_q, d_k, d_v, d_out, M, n_heads, n_kv_heads, n_keys, pos0, S(stream)));
}

int w4a32_op_matmul_f32_nt(const float* d_a, const float* d_b, float* d_c, int M, int N, int K, void* stream) {
  if (!d_a || !d_b || !d_c || M <= 0 || N <= 0 || K <= 0) return W4A32_EINVAL;
  if (K % 4 != 0) return W4A32_ESHAPE;
  if (!aligned16(d_a) || !aligned16(d_b)) return W4A32_EINVAL;
  return from_hip(w4::launch_matmul_f32_nt(d_a, d_b, d_c, M, N, K, S(stream)));
}

int w4a32_op_matmul_nt(const float* d_a, const void* d_b, int b_dtype, float* d_c, int M, int N, int K,
                       void* stream) {
  if (!d_a || !d_b || !d_c || M <= 0 || N <= 0 || K <= 0) return W4A32_EINVAL;
  if (b_dtype != W4A32_DENSE_F32 && b_dtype != W4A32_DENSE_F16) return W4A32_EINVAL;
  if (K % 4 != 0) return W4A32_ESHAPE;
  if (!aligned16(d_a) || !aligned16(d_b)) return W4A32_EINVAL;
  return from_hip(w4::launch_matmul_nt(d_a, d_b, b_dtype, d_c, M, N, K, S(stream)));
}

int w4a32_op_f16_to_f32(const void* d_in, float* d_out, size_t n, void* stream) {
  if (!d_in || !d_out || n == 0) return W4A32_EINVAL;
  if ((reinterpret_cast<uintptr_t>(d_in) & 1) != 0 || (reinterpret_cast<uintptr_t>(d_out) & 3) != 0) return W4A32_EINVAL;
  return from_hip(w4::launch_f16_to_f32(d_in, d_out, n, S(stream)));
}

}  // extern "C"
