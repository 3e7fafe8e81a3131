/*
 * C ABI of the MI355X (gfx950) implementation of mllm-advanced's W4A32 quantized
 * Linear: f32 activations, quantized per row to asymmetric int8 at run time, times
 * 4-bit symmetric block-32 weights with bf16 block scales, f32 output
 * (the reference's KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk).
 *
 * Every pointer named d_* is DEVICE memory on the current HIP device; `stream` is a
 * hipStream_t passed as void* (NULL = the null stream). Calls only enqueue work on
 * `stream` and return; none of them synchronises, allocates or frees. Return value:
 * W4A32_OK or a negative W4A32_E* code - never exit().
 *
 * Each entry point names the reference interface it stands in for (paths relative to
 * the reference tree).
 */
#ifndef W4A32_HIP_H
#define W4A32_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  W4A32_OK = 0,
  W4A32_EINVAL = -1,   /* null pointer, non-positive dimension, misaligned pointer */
  W4A32_ESHAPE = -2,   /* K not a multiple of 32, or M outside the kernel's range */
  W4A32_ELAUNCH = -3,  /* the HIP runtime refused the launch (see hipGetLastError) */
  W4A32_ENOTSUP = -4,  /* request needs a path this build does not provide */
  W4A32_ETOOBIG = -5   /* w4a32_matmul_static_ws: the rows need more than W4A32_STATIC_WS_BYTES */
};

#define W4A32_BLOCK_LEN 32          /* k per weight scale (kai_linear.cpp:328 passes 32) */
#define W4A32_GEMV_MAX_M 8          /* largest M served by the decode (GEMV) kernels */

/* bf16 rounding of the block scale: 0 = truncate (the reference's shipped build: no +bf16
 * arch flag, tests/Arm/KaiLinearTest.hpp:138-139), 1 = round to nearest even (bfcvt). */
#define W4A32_BF16_TRUNC 0
#define W4A32_BF16_RNE 1

const char* w4a32_error_string(int code);

/* Library/version probe; also the symbol a loader checks first. */
int w4a32_abi_version(void);

/* ---- sizes ------------------------------------------------------------------------ */

/* Bytes of the device weight blob for an [N][K] Linear.
 * Replaces KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk::quant_pack_rhs_size
 * (mllm/Backends/Arm/Kernels/kai_linear.cpp:302-309). 0 on invalid shape. */
size_t w4a32_packed_bytes(int N, int K);

/* Bytes of the per-call activation workspace for M rows.
 * Replaces ...::workspace_size (kai_linear.cpp:293-300), called at
 * mllm/Backends/Arm/Ops/LinearOp.cpp:74-78. 0 on invalid shape. */
size_t w4a32_workspace_bytes(int M, int K);

/* Bytes of the row-major 4-bit plane ([N][K/2]) and of the bf16 scale plane ([N][K/32])
 * (get_rhs_native_stride / get_rhs_scale_stride, kai_linear.cpp:317-318). */
size_t w4a32_native_u4_bytes(int N, int K);
size_t w4a32_native_scale_bytes(int N, int K);

/* ---- offline: weights -------------------------------------------------------------- */

/* f32 weights [N][K] row-major -> row-major offset-8 nibbles (even k in the low nibble)
 * + bf16 block scales. Bit-exact restatement of
 * ...::quant_nxk_qs4c32_f32 (kai_linear.cpp:220-291). */
int w4a32_quant_rhs_native(const float* d_w, int N, int K, uint8_t* d_u4, uint16_t* d_scales,
                           int bf16_mode, void* stream);

/* Row-major nibbles + scales (+ optional f32 bias [N], may be NULL) -> the device blob:
 * 16-row x 128-k tiles laid out for 128-bit per-lane loads, block scales beside each
 * tile, then per-row sums and bias. Takes the place of the
 * kai_run_rhs_pack_nxk_qsi4c32p_qsu4c32s1s0 call (kai_linear.cpp:331-344). */
int w4a32_repack_native(const uint8_t* d_u4, const uint16_t* d_scales, const float* d_bias, int N,
                        int K, void* d_packed, void* stream);

/* Both steps at once = ...::quant_pack_rhs_offline (kai_linear.cpp:311-348).
 * d_tmp: scratch of w4a32_native_u4_bytes + w4a32_native_scale_bytes (u4 first). */
int w4a32_quant_pack_rhs(const float* d_w, const float* d_bias, int N, int K, void* d_packed,
                         void* d_tmp, int bf16_mode, void* stream);

/* Inverse of w4a32_repack_native (d_bias may be NULL): recovers the row-major planes
 * bit for bit. No counterpart in the reference (KleidiAI has no unpack); it exists so the
 * layout can be checked and so blobs can be exported. */
int w4a32_unpack_native(const void* d_packed, int N, int K, uint8_t* d_u4, uint16_t* d_scales,
                        float* d_bias, void* stream);

/* Blob -> f32 [N][K]: (u4 - 8) * f32(scale), the format's definition of a weight
 * (tests/Arm/KaiLinearTest.hpp:355-361 unpack, :340 scale). */
int w4a32_dequant(const void* d_packed, int N, int K, float* d_out, void* stream);

/* PARITY UNPINNED. The weight blob that the reference's Arm quantizer stores in a .mllm file
 * (KaiQuantizationPass.cpp:172-184: the output of kai_run_rhs_pack_nxk_qsi4c32p_qsu4c32s1s0 called
 * at kai_linear.cpp:331-344) back to the native arrays of w4a32_repack_native(), so that such a
 * file loads without re-quantising. nr, kr, sr are the tile's (nr 4 or 8; kr/sr 8 for the
 * ...p4x8 / ...p8x8 tiles, 4 for ...p4x4). The packing routine is KleidiAI's, which the reference
 * tree does not contain: the layout is restated from its published loop and checked only against
 * this repository's own restatement (oracle/kai_blob.py).
 * w4a32_kai_blob_bytes(): ceil(N/nr)*nr * (K/32 * 18 + 8), what quant_pack_rhs_size returns
 * (kai_linear.cpp:302-309); 0 for an unsupported shape. d_bias may be NULL. */
size_t w4a32_kai_blob_bytes(int N, int K, int nr);
int w4a32_unpack_kai(const void* d_kai_blob, int N, int K, int nr, int kr, int sr, uint8_t* d_u4,
                     uint16_t* d_scales, float* d_bias, void* stream);

/* ---- online: one forward ------------------------------------------------------------ */

/* Per-row asymmetric int8 quantisation of the activations into the workspace
 * (scale, offset, int8 values), bit-exact with the scalar model
 * tests/Arm/KaiLinearTest.hpp:163-230. Replaces the kai_run_lhs_quant_pack_qai8dxp_f32
 * call (kai_linear.cpp:358-362). ldx = row stride of d_x in elements. */
int w4a32_quant_lhs(const float* d_x, int M, int K, int ldx, void* d_ws, void* stream);

/* Copies the quantised rows out of a workspace for inspection: int8 [M][K], f32 [M]
 * reciprocal scale, i32 [M] negated zero point (the row header of KaiLinearTest.hpp:208-214). */
int w4a32_export_lhs(const void* d_ws, int M, int K, int8_t* d_aq, float* d_recip_scale,
                     int32_t* d_neg_zero_point, void* stream);

/* y[M][N] = clamp(lhs_scale * sum_b scale_b * sum_k (a_q + off) * q  + bias) on rows already
 * quantised into d_ws. M <= W4A32_GEMV_MAX_M: decode kernels; larger M: prefill kernels.
 * Replaces the tile loop + ukernel.run_matmul of ...::matmul (kai_linear.cpp:364-397). */
int w4a32_matmul_quantized(float* d_y, const void* d_ws, const void* d_packed, int M, int K, int N,
                           void* stream);

/* Same product with the kernel named by the caller (tests and benchmarks compare them).
 * The reference picks its micro-kernel the same way, by a tile id argument
 * (KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk::Tiles, kai_linear.hpp:76-118). */
#define W4A32_KERNEL_AUTO 0       /* M <= 8: GEMV, else f16 MFMA */
#define W4A32_KERNEL_GEMV 1       /* v_dot4 decode kernel, M <= 8 */
#define W4A32_KERNEL_GEMM_I8 2    /* int8 MFMA, exact int32 block sums, any M */
#define W4A32_KERNEL_GEMM_F16 3   /* f16 MFMA on exact f16 operands, M > 8; tile shape by size */
/* The f16 kernel with one named tile shape, W4A32_KERNEL_GEMM_F16_TILE0 + i:
 * i = 0: 64 x 64, 1: 128 x 64, 2: 128 x 128, 3: 256 x 128 (rows x columns per workgroup),
 * 4: 128 x 64 with one barrier per two stages, 5: 128 x 160, 6: 128 x 128 with eight wavefronts (each
 * 32-k half of a stage has its own four), 7: 256 x 96, 8: 256 x 96 with one barrier per two stages,
 * 9: 256 x 128 with one barrier per two stages. */
#define W4A32_KERNEL_GEMM_F16_TILE0 16
#define W4A32_GEMM_F16_TILES 10
int w4a32_matmul_quantized_ex(float* d_y, const void* d_ws, const void* d_packed, int M, int K,
                              int N, int kernel, void* stream);

/* The same product for callers that can lend scratch memory: when the problem has few output
 * tiles and a long K (down_proj at prefill sizes) each tile's k range is dealt to several
 * workgroups, which leave partial sums in d_scratch; a second kernel adds them in a fixed order.
 * w4a32_splitk_scratch_bytes() returns the bytes this needs, 0 when the library would not split the
 * shape; with less scratch than that the call is w4a32_matmul_quantized(). The reference has no
 * counterpart: its matmul splits M over threads only (kai_linear.cpp:366-396). */
size_t w4a32_splitk_scratch_bytes(int M, int K, int N);
int w4a32_matmul_quantized_splitk(float* d_y, const void* d_ws, const void* d_packed, int M, int K,
                                  int N, void* d_scratch, size_t scratch_bytes, void* stream);

/* The whole op = ...::matmul (kai_linear.cpp:350-398): quantise rows of d_x into d_ws,
 * then multiply. d_ws must hold w4a32_workspace_bytes(M, K). */
int w4a32_matmul(float* d_y, const float* d_x, const void* d_packed, void* d_ws, int M, int K,
                 int N, void* stream);

/* The whole op for a caller that says how large its workspace is: with at least w4a32_workspace_bytes_n(M, K, N)
 * bytes at d_ws (the activation workspace plus, behind it, room for the partial sums of a product whose k range
 * the library deals to several workgroups: down_proj at prefill sizes) the call takes that faster form itself;
 * with at least w4a32_workspace_bytes(M, K) it is w4a32_matmul; with less, W4A32_EINVAL. One call per Linear,
 * as ...::matmul (kai_linear.cpp:350-398) is called from ArmLinearOp::forward
 * (mllm/Backends/Arm/Ops/LinearOp.cpp:67-83), whose workspace_size() this pair replaces. Results equal
 * w4a32_matmul_quantized_splitk's where the k range is split (f32 rounding of the parts' sum apart from
 * w4a32_matmul's), else w4a32_matmul's bit for bit. */
size_t w4a32_workspace_bytes_n(int M, int K, int N);
int w4a32_matmul_ws(float* d_y, const float* d_x, const void* d_packed, void* d_ws, size_t ws_bytes, int M,
                    int K, int N, void* stream);

/* w4a32_matmul without a workspace argument, for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops and harnesses that forbid hipMalloc). It has no counterpart in the
 * reference, whose forward allocates its workspace on every call (mllm/Backends/Arm/Ops/LinearOp.cpp:74-78).
 * The quantised rows go to a W4A32_STATIC_WS_BYTES array that is part of the library's device code: every
 * GPU the library runs on holds one copy until the process ends, and the call allocates and frees
 * nothing. Same kernels and results as w4a32_matmul, bit for bit.
 *   - W4A32_ETOOBIG when w4a32_workspace_bytes(M, K) exceeds W4A32_STATIC_WS_BYTES (16 MiB: M = 512 rows
 *     of K = 8960, or 3600 rows of K = 1536); nothing is launched then.
 *   - All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race.
 *     Calls on one stream are ordered and need nothing more. The array keeps the last call's rows: a
 *     call overwrites the M rows it multiplies, and what the product kernels read beyond them (up to 31
 *     rows of padding) only feeds output rows that are never stored.
 *   - The first call on a device looks the array's address up (hipGetSymbolAddress); make that call outside
 *     stream capture. A first call on a stream that is capturing returns W4A32_ENOTSUP and launches nothing
 *     (the capture stays valid); after one call outside capture the same call captures and replays. */
#define W4A32_STATIC_WS_BYTES (16u << 20)
int w4a32_matmul_static_ws(float* d_y, const float* d_x, const void* d_packed, int M, int K, int N,
                           void* stream);

/* Several Linears applied to the SAME activation rows, in one launch where the sizes allow:
 * d_y, d_packed and N are HOST arrays of `count` (<= W4A32_MAX_GROUP) entries; Linear i has blob
 * d_packed[i] for [N[i]][K] and writes d_y[i][M][N[i]]. Stands in for the consecutive matmul
 * calls the model code makes on one input - q_proj/k_proj/v_proj and gate_proj/up_proj
 * (mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:47-54, 106-155) - each of which would otherwise
 * quantise the same rows again (kai_linear.cpp:358-362). Results are bit-identical to calling
 * w4a32_matmul once per Linear. */
#define W4A32_MAX_GROUP 4
int w4a32_matmul_grouped(float* const* d_y, const float* d_x, const void* const* d_packed,
                         const int* N, int count, void* d_ws, int M, int K, void* stream);

/* The grouped product on rows that are already quantised into d_ws (w4a32_quant_lhs or one of the
 * fused quantisers of w4a32_decoder.h): at M > 8 one launch of the prefill kernel over all the
 * Linears, else one product per Linear. */
int w4a32_matmul_quantized_grouped(float* const* d_y, const void* d_ws, const void* const* d_packed,
                                   const int* N, int count, int M, int K, void* stream);

/* d_act[M][N] = silu(x W_gate^T + b_gate) * (x W_up^T + b_up) on rows already quantised into d_ws, M > 8:
 * the MLP's gate_proj, up_proj, SiLU and multiply (modeling_ds_qwen2.hpp:47-54) in one launch of the
 * prefill kernel. A wavefront computes both Linears for the same outputs and stores only their product,
 * so neither Linear's [M][N] result is written or read back. Each factor is the value
 * w4a32_matmul_quantized gives (same products and summation order), combined with w4a32_op_silu_mul's
 * expression. W4A32_ESHAPE for M <= 8. */
int w4a32_matmul_quantized_silu_pair(float* d_act, const void* d_ws, const void* d_gate, const void* d_up,
                                     int M, int K, int N, void* stream);

#ifdef __cplusplus
}
#endif
#endif
