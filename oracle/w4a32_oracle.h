/*
 * CPU oracle for the W4A32 quantized Linear (f32 activations quantized per row
 * to asymmetric int8, 4-bit symmetric block-32 weights with bf16 scales, f32 out).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. Only the tests, the smoke
 * check and the benchmark's CPU-baseline leg may call it; the shipped library
 * never links or loads it.
 *
 * It restates, in scalar C, the arithmetic the reference holds for this path:
 *   tests/Arm/KaiLinearTest.hpp:133-149   bf16 <-> f32 casts
 *   tests/Arm/KaiLinearTest.hpp:154-161   uniform[-1,1] input generator (glibc rand)
 *   tests/Arm/KaiLinearTest.hpp:163-230   per-row asymmetric int8 activation quant
 *   mllm/Backends/Arm/Kernels/kai_linear.cpp:220-291  4-bit block-32 weight quant
 *   tests/Arm/KaiLinearTest.hpp:311-385   integer block dot + f32 block scaling
 *   mllm/Backends/Arm/Kernels/kai_linear.cpp:311-348  bias travels with the weight
 *   mllm/Backends/Arm/Kernels/kai_linear.cpp:386-393  clamp to [-FLT_MAX, FLT_MAX]
 *
 * The micro-kernel the reference actually runs lives in KleidiAI (git submodule
 * mllm/Backends/Arm/Vendors/kleidiai, not vendored, pin unknown); the reference's
 * own test asserts that kernel equals the scalar model restated here to 1e-4.
 *
 * Pinning status (each is checked in tests/test_oracle_*.py against closed
 * forms, invariants, brute force and library routines - not against a retyped
 * copy of itself):
 *   orc_bf16_*            pinned (closed form: u32>>16; RNE vs torch.bfloat16)
 *   orc_quant_rhs_qs4c32  pinned (constant / one-hot / zero / negated blocks,
 *                         tie rule, nibble order, reconstruction bound)
 *   orc_quant_lhs_qa8dx   pinned (zero row, one-sided rows, symmetric row ->
 *                         RNE zero point, error bound, clamp)
 *   orc_matmul            pinned (exactly-representable inputs == numpy matmul,
 *                         K=32 brute force, row linearity, bias closed form)
 *   orc_linear_w4a32      the whole op (row quantiser, block dots, scales, bias,
 *                         clamp) pinned bit for bit against a routine written
 *                         elsewhere: PyTorch's aten::_dyn_quant_matmul_4bit
 *                         (block 32, bf16 scales), whose portable C++ path is the
 *                         Arm kernels' authors' own reference for this scheme -
 *                         random rows with outliers, the quantiser's corner rows
 *                         and the reference test's srand() inputs.
 *   the adding of bias    "+bias[n] after the lhs scale": closed form, and equal
 *                         to PyTorch's routine above. The reference test passes no
 *                         bias, so the Arm kernel itself is not observed adding it.
 */
#ifndef W4A32_ORACLE_H
#define W4A32_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_BLOCK_LEN 32

/* KaiLinearTest.hpp:133-142 (non-BF16 build: truncation) and the bfcvt branch (RNE). */
uint16_t orc_bf16_from_f32_trunc(float v);
uint16_t orc_bf16_from_f32_rne(float v);
/* KaiLinearTest.hpp:144-149 */
float orc_f32_from_bf16(uint16_t v);

/* KaiLinearTest.hpp:154-161: srand(seed); (float)((double)rand()/RAND_MAX)*2-1 */
void orc_fill_uniform_random(size_t num_rows, size_t num_cols, float* dst, size_t seed);

/* helpers, KaiLinearTest.hpp:300-309 */
size_t orc_num_blocks_per_row(size_t k, size_t bl);
size_t orc_rhs_native_stride(size_t k);              /* bytes of u4 per weight row */
size_t orc_lhs_row_stride(size_t k);                 /* bytes per quantized activation row */

/* kai_linear.cpp:220-291. rhs_f32 [n][k] row-major -> rhs_u4 [n][ceil(k/2)]
 * (offset-8 nibbles, even k in the low nibble) and scales [n][ceil(k/bl)] bf16.
 * bf16_rne = 0 reproduces the shipped build (no +bf16 arch flag => truncation). */
void orc_quant_rhs_qs4c32(size_t n, size_t k, size_t bl, const float* rhs_f32,
                          uint8_t* rhs_u4, uint16_t* scales_bf16, int bf16_rne);

/* KaiLinearTest.hpp:163-230. Row layout: f32 recip_scale, i32 (-zero_point), k x i8. */
void orc_quant_lhs_qa8dx(size_t m, size_t k, const float* lhs_f32, size_t lhs_stride_elems,
                         int8_t* lhs_qa8dx);

/* KaiLinearTest.hpp:311-385 plus "+ bias[n]" (nullable) before the clamp. */
void orc_matmul_qa8dx_qs4c32(size_t m, size_t n, size_t k, size_t bl, const int8_t* lhs_qa8dx,
                             const uint8_t* rhs_u4, const uint16_t* scales_bf16,
                             const float* bias, float* dst_f32, float scalar_min,
                             float scalar_max, int num_threads);

/* (u4 - 8) * f32(scale) for every weight: what "dequant" means for this format. */
void orc_dequant_qs4c32(size_t n, size_t k, size_t bl, const uint8_t* rhs_u4,
                        const uint16_t* scales_bf16, float* out_f32);

/* Whole op on already-quantized weights: quantize rows of x, then matmul. */
void orc_linear_w4a32(size_t m, size_t n, size_t k, const float* x, const uint8_t* rhs_u4,
                      const uint16_t* scales_bf16, const float* bias, float* y, int num_threads);

/*
 * w4a32_oracle_vnni.c: orc_matmul_qa8dx_qs4c32 / orc_linear_w4a32 with the block dots on AVX-512
 * VNNI (bl = 32, k % 32 == 0), bit-identical results; for the benchmark's CPU-baseline leg.
 * Return 0, or -1 when the CPU lacks AVX-512 VNNI (orc_has_avx512_vnni() == 0) or k does not fit.
 */
int orc_has_avx512_vnni(void);
int orc_matmul_qa8dx_qs4c32_vnni(size_t m, size_t n, size_t k, const int8_t* lhs_qa8dx,
                                 const uint8_t* rhs_u4, const uint16_t* scales_bf16,
                                 const float* bias, float* dst_f32, float scalar_min,
                                 float scalar_max, int num_threads);
int orc_linear_w4a32_vnni(size_t m, size_t n, size_t k, const float* x, const uint8_t* rhs_u4,
                          const uint16_t* scales_bf16, const float* bias, float* y, int num_threads);

#ifdef __cplusplus
}
#endif
#endif
