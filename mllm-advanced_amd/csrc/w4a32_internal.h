// Launchers behind the C ABI. Each returns hipError_t of the launch; arguments are already
// validated by the caller (w4a32_capi.hip).
#pragma once

#include <atomic>
#include <hip/hip_runtime.h>

#include "w4a32_hip.h"
#include "w4a32_layout.h"

namespace w4 {

// weights (offline)
hipError_t launch_quant_rhs(const float* w, int N, int K, uint8_t* u4, uint16_t* scales, int rne,
                            hipStream_t s);
hipError_t launch_repack(const uint8_t* u4, const uint16_t* scales, const float* bias, int N, int K,
                         uint8_t* packed, hipStream_t s);
hipError_t launch_unpack(const uint8_t* packed, int N, int K, uint8_t* u4, uint16_t* scales,
                         float* bias, hipStream_t s);
hipError_t launch_dequant(const uint8_t* packed, int N, int K, float* out, hipStream_t s);
// blob of the reference's Arm quantizer (KleidiAI packing, parity unpinned) -> native arrays
hipError_t launch_unpack_kai(const uint8_t* blob, int N, int K, int nr, int kr, int sr, uint8_t* u4,
                             uint16_t* scales, float* bias, hipStream_t s);

// activations (every forward)
hipError_t launch_quant_lhs(const float* x, int M, int K, int ldx, uint8_t* ws, hipStream_t s);
// the quantiser with the operator that produces its rows in front (prefill sizes): residual add +
// RMSNorm, or silu(gate) * up; K must satisfy quant_rows_fusable()
bool quant_rows_fusable(int K);
hipError_t launch_quant_lhs_norm(const float* h, const float* delta, const float* norm_w, float eps,
                                 float* h_out, int M, int K, uint8_t* ws, hipStream_t s);
// ... with delta = ((parts[0] + parts[1]) + ...) + bias, parts = [nparts][M][K] as launch_gemm_splitk leaves
// them when it is given no output
hipError_t launch_quant_lhs_norm_parts(const float* h, const float* parts, int nparts, const float* bias,
                                       const float* norm_w, float eps, float* h_out, int M, int K,
                                       uint8_t* ws, hipStream_t s);
hipError_t launch_quant_lhs_silu_mul(const float* gate, const float* up, int M, int K, uint8_t* ws,
                                     hipStream_t s);

// products
hipError_t launch_gemv(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                       hipStream_t s);
// whole decode op in one launch (row quantisation inside the product kernel)
bool gemv_fused_applies(int M, int K, int N);
hipError_t launch_gemv_fused(float* y, const float* x, int ldx, const uint8_t* packed, int M, int K,
                             int N, hipStream_t s);
// several Linears on the same activation rows in one launch (decode sizes only)
bool gemv_group_applies(int M, int K, const int* N, int count);
hipError_t launch_gemv_group(float* const* y, const float* x, int ldx, const uint8_t* const* packed,
                             const int* N, int count, int M, int K, hipStream_t s);
// one decode row through 1..4 Linears, optionally with (residual add +) RMSNorm in front and
// silu(y0) * y1 behind
bool gemv_decode_applies(int K, const int* N, int count, bool pair);
// in_parts > 1: the row (the delta row when there is a norm) is the sum of that many rows, K floats apart
hipError_t launch_gemv_decode(float* const* y, const float* x, const uint8_t* const* packed,
                              const int* N, int count, int K, const float* delta, float* sum_out,
                              const float* norm_w, float eps, bool pair, int in_parts, hipStream_t s,
                              const int64_t* x_row = nullptr, int x_rows = 0, float* amax_val = nullptr,
                              int* amax_idx = nullptr);
// lm_head-sized Linears (one wavefront per tile row): does that kernel take [N][K], and how many wavefronts
// (partial argmax results, see launch_gemv_decode's amax_val / amax_idx) does its launch have
bool gemv_wide_applies(int K, int N);
int wide_partials(int N);
// one decode row through one Linear with its k range dealt to gemv_kparts(K, N) workgroups per tile row, the
// result left as that many partial rows y_parts[p][N] for the reader to add up (1: the shape is not split)
int gemv_kparts(int K, int N);
hipError_t launch_gemv_kparts(float* y_parts, const float* x, const uint8_t* packed, int K, int N,
                              hipStream_t s);
hipError_t launch_gemm(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                       int kernel, hipStream_t s);
// the f16 kernel with every tile's k range dealt to several workgroups (partial sums in `part`,
// which holds parts * M * N floats), then a reduction; for few tiles and a long K
// A kernel that needs more dynamic LDS than the default limit has the limit raised once per device
// (the attribute belongs to the function on the current device); bit d of the mask = done on device d.
struct LdsLimitOnce {
  std::atomic<unsigned long long> done{0};
  hipError_t raise(const void* kernel, size_t bytes) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    const unsigned long long bit = dev < 64 ? 1ull << dev : 0;  // past 64 devices: set on every call
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    if (hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        e != hipSuccess)
      return e;
    done.fetch_or(bit, std::memory_order_release);
    return hipSuccess;
  }
};

struct SplitPlan {
  int tile, parts;
};
SplitPlan splitk_plan(int M, int K, int N);
hipError_t launch_gemm_pair(float* act, const uint8_t* ws, const uint8_t* gate, const uint8_t* up, int M,
                            int K, int N, hipStream_t s);
const float* linear_bias(const uint8_t* packed, int N, int K);  // the bias row inside a packed blob
hipError_t launch_gemm_splitk(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                              float* part, hipStream_t s);
// several Linears on the same quantised rows in one launch of the f16 kernel (M > 8)
hipError_t launch_gemm_group(float* const* y, const uint8_t* ws, const uint8_t* const* packed,
                             const int* N, int count, int M, int K, hipStream_t s);

// decoder operators (f32), w4a32_glue.hip
hipError_t launch_embedding(const int64_t* ids, const float* table, int M, int D, int vocab,
                            float* out, hipStream_t s);
hipError_t launch_rmsnorm(const float* h, const float* delta, const float* w, int M, int D, float eps,
                          float* h_out, float* y, hipStream_t s);
hipError_t launch_add(const float* a, const float* b, float* out, size_t n, hipStream_t s);
hipError_t launch_silu_mul(const float* g, const float* u, float* out, size_t n, hipStream_t s);
hipError_t launch_rope_table(float* sin_t, float* cos_t, int max_pos, int D, float base, hipStream_t s);
hipError_t launch_rope_kv(float* q, const float* k, const float* v, const float* sin_t,
                          const float* cos_t, float* kc, float* vc, int M, int Hq, int Hkv, int D,
                          int max_seq, const int* d_pos0, int pos0, hipStream_t s);
size_t attention_prefill_part_bytes(int M, int Hq);
hipError_t launch_attention_prefill(const float* q, const float* kc, const float* vc, float* out,
                                    int M, int Hq, int Hkv, int max_seq, const int* d_pos0, int pos0,
                                    float* part, size_t part_bytes, unsigned int* counters, hipStream_t s);
// the same operator with its products on the bf16 matrix pipe, every f32 operand as three bf16 terms
// (w4a32_attention16.hip); scratch: attention16_scratch_bytes(pos0 + M, Hkv) bytes, 16-byte aligned
size_t attention16_scratch_bytes(int n_keys, int Hkv);
hipError_t launch_attention16(const float* q, const float* kc, const float* vc, float* out, int M, int Hq, int Hkv,
                              int max_seq, int pos0, uint8_t* scratch, hipStream_t s);
// launch_rope_kv at a position known on the host + launch_attention16, with the rotation, the cache append and the
// operand split in one launch (head_dim 128)
hipError_t launch_rope_attention16(float* q, const float* k, const float* v, const float* sin_t,
                                   const float* cos_t, float* kc, float* vc, float* out, int M, int Hq, int Hkv,
                                   int max_seq, int pos0, uint8_t* scratch, hipStream_t s);
hipError_t launch_attention_bshd(const float* q, const float* k, const float* v, float* out, int M, int Hq,
                                 int Hkv, int n_keys, int pos0, hipStream_t s);
// operators of the engine's op-by-op path (w4a32_engine_ops.hip)
hipError_t launch_silu(const float* x, float* out, size_t n, hipStream_t s);
hipError_t launch_mul(const float* a, const float* b, float* out, size_t n, hipStream_t s);
hipError_t launch_rope_rows(const float* x, float* y, const float* sin_t, const float* cos_t, int M, int H,
                            int D, int pos0, hipStream_t s);
hipError_t launch_matmul_f32_nt(const float* a, const float* b, float* c, int M, int N, int K, hipStream_t s);
// dense [N][K] operands held as f16 or f32 (b_dtype: W4A32_DENSE_*), w4a32_dense.hip
hipError_t launch_matmul_nt(const float* a, const void* b, int b_dtype, float* c, int M, int N, int K, hipStream_t s);
hipError_t launch_f16_to_f32(const void* in, float* out, size_t n, hipStream_t s);
bool dense_rows_applies(int M, int K);  // M <= 8 rows against a streamed B
int dense_rows_partials(int N);         // wavefronts (= partial argmax results) of such a launch at M = 1
hipError_t launch_dense_rows(const float* x, int ldx, const void* b, int b_dtype, float* c, int M, int N, int K,
                             hipStream_t s);
// one decode row through a dense lm_head with the residual add (delta_parts partial rows, or none) and the
// RMSNorm in front; optionally one (max, first column) pair per wavefront to amax_val / amax_idx
hipError_t launch_dense_head(const float* h, const float* delta, int delta_parts, const float* norm_w, float eps,
                             const void* b, int b_dtype, float* logits, int N, int K, float* amax_val,
                             int* amax_idx, hipStream_t s);
hipError_t launch_attention_decode(const float* q, float* kc, float* vc, float* out, int Hq, int Hkv,
                                   int max_seq, const int* d_pos0, int pos0, int nsplit, float* part,
                                   unsigned int* counters, const float* k_new, const float* v_new,
                                   const float* sin_t, const float* cos_t, bool defer, hipStream_t s);
// one decode row through one Linear whose input row is still in key slices, as the decode attention leaves it
// with defer = true (`part`: the same pointer, `slices`: its nsplit)
bool gemv_attn_rows_applies(int K, int N, int slices);
hipError_t launch_gemv_attn_rows(float* y, const float* part, int slices, const uint8_t* packed, int K, int N,
                                 hipStream_t s);
hipError_t launch_argmax(const float* logits, int n, float* part_val, int* part_idx,
                         unsigned int* counter, int64_t* token_out, int* pos_to_advance, int blocks,
                         hipStream_t s);
hipError_t launch_argmax_parts(const float* val, const int* idx, int n, int64_t* token_out, int* pos_to_advance,
                               hipStream_t s);
hipError_t launch_im2col_conv3d(const float* a, float* z, int B, int C, int T, int H, int W, int kt,
                                int kh, int kw, int st, int sh, int sw, int ld, hipStream_t s);
hipError_t launch_set_int(int* p, int value, hipStream_t s);
hipError_t launch_add_to_int(int* p, int delta, hipStream_t s);
hipError_t launch_zero_u32(unsigned int* p, int n, hipStream_t s);

// kernel selectors of w4a32_matmul_quantized_ex (0 = the library's own choice)
constexpr int kKernelAuto = 0;
constexpr int kKernelGemv = 1;
constexpr int kKernelGemmI8 = 2;
constexpr int kKernelGemmF16 = 3;
constexpr int kKernelGemmF16Tile = W4A32_KERNEL_GEMM_F16_TILE0;  // + index: that tile shape
constexpr int kGemmF16Tiles = W4A32_GEMM_F16_TILES;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// Loads and stores through pointers picked from the group table must say that they address global
// memory: the compiler no longer knows, would emit flat instructions and, because those may
// complete out of order with global ones, wait for every outstanding load at the first use of any.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define W4_GLOBAL __attribute__((address_space(1)))
// silu(g) * u = g / (1 + e^-g) * u, the one expression every kernel that applies the MLP's activation
// uses (the standalone operator, the row quantiser that applies it on the way, the decode pair kernel and
// the prefill pair kernel's epilogue), so that they agree bit for bit. Hardware exponential and
// reciprocal (about 1 ulp each): where the activation runs in a product kernel's epilogue, on a few
// wavefronts per CU, the correctly rounded library routines cost as much as the products of a tile.
__device__ __forceinline__ float silu_mul(float g, float u) {
  const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
  return g * __builtin_amdgcn_rcpf(1.0f + e) * u;
}

template <typename T>
__device__ __forceinline__ T load_global(const void* p) {
  return *(const W4_GLOBAL T*)p;
}


}  // namespace w4
