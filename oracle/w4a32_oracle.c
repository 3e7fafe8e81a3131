/*
 * Scalar CPU oracle for the W4A32 quantized Linear. Test infrastructure only:
 * see w4a32_oracle.h for what it restates and how each function is pinned.
 *
 * Build with -ffp-contract=off: every f32 product below must be rounded before
 * it is used (the reference rounds x*scale to f32, then calls round()).
 */
#include "w4a32_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

static inline uint32_t f32_bits(float v) {
  uint32_t u;
  memcpy(&u, &v, sizeof u);
  return u;
}

static inline float bits_f32(uint32_t u) {
  float v;
  memcpy(&v, &u, sizeof v);
  return v;
}

/* tests/Arm/KaiLinearTest.hpp:138-139: keep the upper 16 bits. */
uint16_t orc_bf16_from_f32_trunc(float v) { return (uint16_t)(f32_bits(v) >> 16); }

/* tests/Arm/KaiLinearTest.hpp:136 (bfcvt): IEEE round-to-nearest-even, NaN kept quiet. */
uint16_t orc_bf16_from_f32_rne(float v) {
  uint32_t u = f32_bits(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) { return (uint16_t)((u >> 16) | 0x0040u); }
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

/* tests/Arm/KaiLinearTest.hpp:144-149 */
float orc_f32_from_bf16(uint16_t v) { return bits_f32((uint32_t)v << 16); }

/* tests/Arm/KaiLinearTest.hpp:154-161 */
void orc_fill_uniform_random(size_t num_rows, size_t num_cols, float* dst, size_t seed) {
  srand((unsigned)seed);
  const size_t total = num_rows * num_cols;
  for (size_t i = 0; i < total; ++i) { dst[i] = (float)((double)rand() / RAND_MAX) * 2 - 1; }
}

size_t orc_num_blocks_per_row(size_t k, size_t bl) { return (k + bl - 1) / bl; }
size_t orc_rhs_native_stride(size_t k) { return (k + 1) / 2; }
size_t orc_lhs_row_stride(size_t k) { return k + sizeof(float) + sizeof(int32_t); }

/*
 * mllm/Backends/Arm/Kernels/kai_linear.cpp:220-291.
 * Per (row, block): pick the first element of largest magnitude, scale = it / -8,
 * q = clamp(round(x * (1/scale)), -8, 7), stored as q+8; even k -> low nibble.
 */
void orc_quant_rhs_qs4c32(size_t n, size_t k, size_t bl, const float* rhs_f32,
                          uint8_t* rhs_u4, uint16_t* scales_bf16, int bf16_rne) {
  const size_t nb = orc_num_blocks_per_row(k, bl);
  const size_t row_bytes = orc_rhs_native_stride(k);
  memset(rhs_u4, 0, n * row_bytes);

  for (size_t r = 0; r < n; ++r) {
    const float* w = rhs_f32 + r * k;
    uint8_t* out = rhs_u4 + r * row_bytes;
    for (size_t b = 0; b < nb; ++b) {
      const size_t k0 = b * bl;
      const size_t k1 = (k0 + bl < k) ? k0 + bl : k;

      float best_abs = 0.0f, best = 0.0f;
      for (size_t i = k0; i < k1; ++i) {
        const float a = fabsf(w[i]);
        if (best_abs < a) { /* strict: the first maximum wins (kai_linear.cpp:248) */
          best_abs = a;
          best = w[i];
        }
      }
      const float scale = (float)(best / -8.0);                 /* kai_linear.cpp:254 */
      const float recip = scale ? 1.0f / scale : 0.0f;          /* kai_linear.cpp:255 */
      scales_bf16[r * nb + b] =
          bf16_rne ? orc_bf16_from_f32_rne(scale) : orc_bf16_from_f32_trunc(scale);

      for (size_t i = k0; i < k1; ++i) {
        const float scaled = w[i] * recip;                      /* f32 product */
        int32_t q = (int32_t)round((double)scaled);             /* half away from zero */
        if (q < -8) q = -8;
        if (q > 7) q = 7;
        const uint8_t u = (uint8_t)(q + 8);
        if ((i & 1u) == 0) {
          out[i >> 1] = u;
        } else {
          out[i >> 1] |= (uint8_t)(u << 4);
        }
      }
    }
  }
}

/*
 * tests/Arm/KaiLinearTest.hpp:163-230. Asymmetric int8, range always contains 0.
 */
void orc_quant_lhs_qa8dx(size_t m, size_t k, const float* lhs_f32, size_t lhs_stride_elems,
                         int8_t* lhs_qa8dx) {
  const size_t out_stride = orc_lhs_row_stride(k);
  for (size_t r = 0; r < m; ++r) {
    const float* x = lhs_f32 + r * lhs_stride_elems;
    float hi = -FLT_MAX, lo = FLT_MAX;
    for (size_t i = 0; i < k; ++i) {
      hi = x[i] > hi ? x[i] : hi; /* NaN inputs are outside the contract of this path */
      lo = x[i] < lo ? x[i] : lo;
    }
    const float qmin = -128.0f, qmax = 127.0f;
    const float rmin = lo < 0.0f ? lo : 0.0f;
    const float rmax = hi > 0.0f ? hi : 0.0f;
    const float scale = (rmin == rmax) ? 1.0f : (qmax - qmin) / (rmax - rmin);
    const float recip = scale ? 1.0f / scale : 0.0f;

    const float dmin = rmin * scale;
    const float dmax = rmax * scale;
    const float err_min = qmin + dmin;
    const float err_max = qmax + dmax;
    float zp = (err_min + err_max > 0.0f) ? (qmin - dmin) : (qmax - dmax);
    zp = zp > qmin ? zp : qmin;
    zp = zp < qmax ? zp : qmax;
    const int32_t zpi = (int32_t)lrintf(zp); /* default rounding mode: nearest even */

    int8_t* out = lhs_qa8dx + r * out_stride;
    const int32_t neg_zp = -zpi;
    memcpy(out, &recip, sizeof recip);
    memcpy(out + sizeof(float), &neg_zp, sizeof neg_zp);
    out += sizeof(float) + sizeof(int32_t);
    for (size_t i = 0; i < k; ++i) {
      const float scaled = x[i] * scale;                        /* f32 product */
      int32_t v = (int32_t)round((double)scaled) + zpi;
      if (v < -128) v = -128;
      if (v > 127) v = 127;
      out[i] = (int8_t)v;
    }
  }
}

/*
 * tests/Arm/KaiLinearTest.hpp:311-385: per block an exact int32 sum of
 * (a_q + lhs_offset) * (u4 - 8), times the block's scale, accumulated in f32 in
 * block order; then * lhs_scale, (+ bias), clamp.
 */
void orc_matmul_qa8dx_qs4c32(size_t m, size_t n, size_t k, size_t bl, const int8_t* lhs_qa8dx,
                             const uint8_t* rhs_u4, const uint16_t* scales_bf16,
                             const float* bias, float* dst_f32, float scalar_min,
                             float scalar_max, int num_threads) {
  const size_t nb = orc_num_blocks_per_row(k, bl);
  const size_t lhs_stride = orc_lhs_row_stride(k);
  const size_t rhs_stride = orc_rhs_native_stride(k);
  if (num_threads < 1) num_threads = 1;

#pragma omp parallel for num_threads(num_threads) schedule(static) collapse(2)
  for (size_t r = 0; r < m; ++r) {
    for (size_t c = 0; c < n; ++c) {
      const int8_t* row = lhs_qa8dx + r * lhs_stride;
      float lhs_scale;
      int32_t lhs_off;
      memcpy(&lhs_scale, row, sizeof lhs_scale);
      memcpy(&lhs_off, row + sizeof(float), sizeof lhs_off);
      const int8_t* a = row + sizeof(float) + sizeof(int32_t);
      const uint8_t* w = rhs_u4 + c * rhs_stride;

      float acc = 0.0f;
      for (size_t b = 0; b < nb; ++b) {
        const size_t k0 = b * bl;
        const size_t k1 = (k0 + bl < k) ? k0 + bl : k;
        int32_t iacc = 0;
        for (size_t i = k0; i < k1; ++i) {
          const uint8_t byte = w[i >> 1];
          const int32_t q = (int32_t)((i & 1u) ? (byte >> 4) : (byte & 0x0f)) - 8;
          iacc += (int32_t)a[i] * q;
          iacc += lhs_off * q;
        }
        acc += (float)iacc * orc_f32_from_bf16(scales_bf16[c * nb + b]);
      }
      acc = acc * lhs_scale;
      if (bias) acc = acc + bias[c];
      acc = acc > scalar_min ? acc : scalar_min;
      acc = acc < scalar_max ? acc : scalar_max;
      dst_f32[r * n + c] = acc;
    }
  }
}

void orc_dequant_qs4c32(size_t n, size_t k, size_t bl, const uint8_t* rhs_u4,
                        const uint16_t* scales_bf16, float* out_f32) {
  const size_t nb = orc_num_blocks_per_row(k, bl);
  const size_t rhs_stride = orc_rhs_native_stride(k);
  for (size_t r = 0; r < n; ++r) {
    for (size_t i = 0; i < k; ++i) {
      const uint8_t byte = rhs_u4[r * rhs_stride + (i >> 1)];
      const int32_t q = (int32_t)((i & 1u) ? (byte >> 4) : (byte & 0x0f)) - 8;
      out_f32[r * k + i] = (float)q * orc_f32_from_bf16(scales_bf16[r * nb + i / bl]);
    }
  }
}

void orc_linear_w4a32(size_t m, size_t n, size_t k, const float* x, const uint8_t* rhs_u4,
                      const uint16_t* scales_bf16, const float* bias, float* y, int num_threads) {
  int8_t* lhs = (int8_t*)malloc(m * orc_lhs_row_stride(k));
  orc_quant_lhs_qa8dx(m, k, x, k, lhs);
  orc_matmul_qa8dx_qs4c32(m, n, k, ORC_BLOCK_LEN, lhs, rhs_u4, scales_bf16, bias, y, -FLT_MAX,
                          FLT_MAX, num_threads);
  free(lhs);
}
