/*
 * AVX-512 VNNI form of the CPU oracle's product (orc_matmul_qa8dx_qs4c32), for the
 * benchmark's CPU-baseline leg: what an x86 host delivers on this path when the block
 * dots run on vpdpbusd instead of a scalar loop. Test infrastructure only, like the rest
 * of this directory; the shipped library never links or loads it.
 *
 * It computes the same expression as the scalar restatement
 * (tests/Arm/KaiLinearTest.hpp:311-385): per block an exact int32 sum of
 * (a_q + lhs_offset) * (u4 - 8), converted to f32, times the block's bf16 scale, added up
 * in block order; then * lhs_scale, (+ bias), clamp. The integer part is regrouped
 *     sum (a + off)(u - 8) = sum a*u - 8*sum a + off*(sum u - 8*32)
 * which is exact in int32 (|a| <= 128, u <= 15, 32 terms), and the f32 part keeps the
 * scalar code's order of operations, so the results are bit-identical to it
 * (tests/test_oracle_pins.py checks that on every shape class).
 *
 * Pinning status: pinned through bit-equality with orc_matmul_qa8dx_qs4c32, which is
 * pinned as w4a32_oracle.h describes.
 */
#include "w4a32_oracle.h"

#include <immintrin.h>
#include <stdlib.h>
#include <string.h>

#define VNNI_TARGET __attribute__((target("avx512f,avx512bw,avx512vl,avx512vnni")))

int orc_has_avx512_vnni(void) {
  __builtin_cpu_init();
  return __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
         __builtin_cpu_supports("avx512vl") && __builtin_cpu_supports("avx512vnni");
}

/* One output: row r's prepared operands against column c's nibbles and scales. */
VNNI_TARGET static inline float vnni_column(size_t nb, const int8_t* a_even, const int8_t* a_odd,
                                            const int32_t* a_sum, int32_t lhs_off,
                                            const uint8_t* w, const uint16_t* scales) {
  const __m512i nib = _mm512_set1_epi8(0x0f);
  const __m512i ones = _mm512_set1_epi8(1);
  const __m512i pick = _mm512_setr_epi32(0, 4, 8, 12, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0);
  const __m128i voff = _mm_set1_epi32(lhs_off);
  float acc = 0.0f;
  for (size_t b = 0; b < nb; b += 4) {
    const size_t left = nb - b < 4 ? nb - b : 4;                 /* blocks in this group */
    const __mmask64 mb = left == 4 ? ~0ull : ((1ull << (16 * left)) - 1);
    const __mmask8 m4 = (__mmask8)((1u << left) - 1);
    const __m512i bytes = _mm512_maskz_loadu_epi8(mb, w + 16 * b);
    const __m512i lo = _mm512_and_si512(bytes, nib);                       /* even k */
    const __m512i hi = _mm512_and_si512(_mm512_srli_epi16(bytes, 4), nib); /* odd k */
    const __m512i ae = _mm512_maskz_loadu_epi8(mb, a_even + 16 * b);
    const __m512i ao = _mm512_maskz_loadu_epi8(mb, a_odd + 16 * b);
    __m512i dot = _mm512_dpbusd_epi32(_mm512_setzero_si512(), lo, ae);
    dot = _mm512_dpbusd_epi32(dot, hi, ao);
    __m512i usum = _mm512_dpbusd_epi32(_mm512_setzero_si512(), lo, ones);
    usum = _mm512_dpbusd_epi32(usum, hi, ones);
    /* a block is 16 bytes = 4 adjacent int32 lanes: add them up inside each 128-bit lane */
    dot = _mm512_add_epi32(dot, _mm512_shuffle_epi32(dot, (_MM_PERM_ENUM)0xB1));
    dot = _mm512_add_epi32(dot, _mm512_shuffle_epi32(dot, (_MM_PERM_ENUM)0x4E));
    usum = _mm512_add_epi32(usum, _mm512_shuffle_epi32(usum, (_MM_PERM_ENUM)0xB1));
    usum = _mm512_add_epi32(usum, _mm512_shuffle_epi32(usum, (_MM_PERM_ENUM)0x4E));
    const __m128i d4 = _mm512_castsi512_si128(_mm512_permutexvar_epi32(pick, dot));
    const __m128i u4 = _mm512_castsi512_si128(_mm512_permutexvar_epi32(pick, usum));
    const __m128i as4 = _mm_maskz_loadu_epi32(m4, a_sum + b);
    /* iacc = dot - 8*sum(a) + off*(sum(u) - 256) */
    __m128i iacc = _mm_sub_epi32(d4, _mm_slli_epi32(as4, 3));
    iacc = _mm_add_epi32(iacc, _mm_mullo_epi32(voff, _mm_sub_epi32(u4, _mm_set1_epi32(8 * ORC_BLOCK_LEN))));
    const __m128i s16 = _mm_maskz_loadu_epi16(m4, scales + b);
    const __m128 sc = _mm_castsi128_ps(_mm_slli_epi32(_mm_cvtepu16_epi32(s16), 16));
    const __m128 prod = _mm_mul_ps(_mm_cvtepi32_ps(iacc), sc);   /* each product rounded to f32 */
    float p[4];
    _mm_storeu_ps(p, prod);
    for (size_t i = 0; i < left; ++i) acc += p[i];               /* block order, as the scalar code */
  }
  return acc;
}

/*
 * Same arguments and results as orc_matmul_qa8dx_qs4c32 with bl = 32 and k a multiple of 32.
 * Returns 0, or -1 (dst untouched) when the CPU lacks AVX-512 VNNI or k is not a multiple of 32.
 */
VNNI_TARGET int orc_matmul_qa8dx_qs4c32_vnni(size_t m, size_t n, size_t k, const int8_t* lhs_qa8dx,
                                             const uint8_t* rhs_u4, const uint16_t* scales_bf16,
                                             const float* bias, float* dst_f32, float scalar_min,
                                             float scalar_max, int num_threads) {
  if (!orc_has_avx512_vnni() || k == 0 || k % ORC_BLOCK_LEN != 0) return -1;
  const size_t nb = k / ORC_BLOCK_LEN;
  const size_t lhs_stride = orc_lhs_row_stride(k);
  const size_t rhs_stride = orc_rhs_native_stride(k);
  if (num_threads < 1) num_threads = 1;

  /* per row: even-k and odd-k values apart (a weight byte holds k = 2i low, 2i+1 high), block sums */
  int8_t* a_even = (int8_t*)malloc(m * k);
  int32_t* a_sum = (int32_t*)malloc(m * nb * sizeof(int32_t));
  if (!a_even || !a_sum) {
    free(a_even);
    free(a_sum);
    return -1;
  }
  int8_t* a_odd = a_even + m * (k / 2);
  for (size_t r = 0; r < m; ++r) {
    const int8_t* a = lhs_qa8dx + r * lhs_stride + sizeof(float) + sizeof(int32_t);
    for (size_t i = 0; i < k / 2; ++i) {
      a_even[r * (k / 2) + i] = a[2 * i];
      a_odd[r * (k / 2) + i] = a[2 * i + 1];
    }
    for (size_t b = 0; b < nb; ++b) {
      int32_t s = 0;
      for (size_t i = 0; i < ORC_BLOCK_LEN; ++i) s += a[b * ORC_BLOCK_LEN + i];
      a_sum[r * nb + b] = s;
    }
  }

#pragma omp parallel for num_threads(num_threads) schedule(static)
  for (size_t c = 0; c < n; ++c) {
    for (size_t r = 0; r < m; ++r) {
      const int8_t* row = lhs_qa8dx + r * lhs_stride;
      float lhs_scale;
      int32_t lhs_off;
      memcpy(&lhs_scale, row, sizeof lhs_scale);
      memcpy(&lhs_off, row + sizeof(float), sizeof lhs_off);
      float acc = vnni_column(nb, a_even + r * (k / 2), a_odd + r * (k / 2), a_sum + r * nb, lhs_off,
                              rhs_u4 + c * rhs_stride, scales_bf16 + c * nb);
      acc = acc * lhs_scale;
      if (bias) acc = acc + bias[c];
      acc = acc > scalar_min ? acc : scalar_min;
      acc = acc < scalar_max ? acc : scalar_max;
      dst_f32[r * n + c] = acc;
    }
  }
  free(a_even);
  free(a_sum);
  return 0;
}

/* The whole op on vpdpbusd: scalar row quantiser (orc_quant_lhs_qa8dx), then the product above. */
int orc_linear_w4a32_vnni(size_t m, size_t n, size_t k, const float* x, const uint8_t* rhs_u4,
                          const uint16_t* scales_bf16, const float* bias, float* y, int num_threads) {
  int8_t* lhs = (int8_t*)malloc(m * orc_lhs_row_stride(k));
  if (!lhs) return -1;
  orc_quant_lhs_qa8dx(m, k, x, k, lhs);
  const int rc = orc_matmul_qa8dx_qs4c32_vnni(m, n, k, lhs, rhs_u4, scales_bf16, bias, y,
                                              -3.402823466e+38f, 3.402823466e+38f, num_threads);
  free(lhs);
  return rc;
}
