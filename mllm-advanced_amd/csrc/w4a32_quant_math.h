// Arithmetic of the per-row asymmetric int8 activation quantiser, shared by the standalone
// row-quant kernel and the decode kernel that quantises its own copy of the activations.
// Bit-exact with the scalar model tests/Arm/KaiLinearTest.hpp:166-228 of the reference: every
// f32 product and sum is an explicitly rounded intrinsic, so no compiler flag can fuse them.
#pragma once

#include <hip/hip_runtime.h>

namespace w4 {

struct RowQuant {
  float scale;   // 255 / (rmax - rmin), or 1 for a constant-zero range
  float recip;   // 1 / scale: the "lhs scale" applied to the output
  int zp;        // zero point in [-128, 127]
};

// lo / hi = min / max over the row (any association: min and max are exact).
__device__ __forceinline__ RowQuant row_quant_params(float lo, float hi) {
  const float qmin = -128.0f, qmax = 127.0f;
  const float rmin = (lo < 0.0f) ? lo : 0.0f;
  const float rmax = (hi > 0.0f) ? hi : 0.0f;
  RowQuant p;
  p.scale = (rmin == rmax) ? 1.0f : __fdiv_rn(255.0f, __fsub_rn(rmax, rmin));
  p.recip = (p.scale != 0.0f) ? __fdiv_rn(1.0f, p.scale) : 0.0f;
  const float dmin = __fmul_rn(rmin, p.scale);
  const float dmax = __fmul_rn(rmax, p.scale);
  const float err_min = __fadd_rn(qmin, dmin);
  const float err_max = __fadd_rn(qmax, dmax);
  float zpf = (__fadd_rn(err_min, err_max) > 0.0f) ? __fsub_rn(qmin, dmin) : __fsub_rn(qmax, dmax);
  zpf = fminf(fmaxf(zpf, qmin), qmax);
  p.zp = __float2int_rn(zpf);  // nearest even, as lrintf in the default rounding mode
  return p;
}

// round_half_away(v) for |v| < 2^23 as trunc(v + copysign(0.5 - 2^-25, v)): below a tie the sum
// stays under the next integer (it is exact or rounds down), at a tie it rounds up to it.
__device__ __forceinline__ float round_half_away(float v) {
  return __builtin_truncf(__fadd_rn(v, __builtin_copysignf(0.49999997f, v)));
}

// round_half_away(x * scale) + zp, clamped to int8. |x * scale| <= 255, so the cast is safe.
__device__ __forceinline__ int quant_one(float x, const RowQuant& p) {
  int r = (int)round_half_away(__fmul_rn(x, p.scale)) + p.zp;
  r = r < -128 ? -128 : r;
  return r > 127 ? 127 : r;
}

__device__ __forceinline__ uint32_t pack4(const int* q) {
  return (uint32_t)(q[0] & 0xFF) | ((uint32_t)(q[1] & 0xFF) << 8) | ((uint32_t)(q[2] & 0xFF) << 16) |
         ((uint32_t)(q[3] & 0xFF) << 24);
}

// Eight consecutive values of a row -> eight int8, packed in memory order. The rounded value plus
// zp + 128 is an integer in f32; v_cvt_pk_u8_f32 saturates it to [0, 255] and drops it into its
// byte, and flipping bit 7 of every byte subtracts the 128 again.
__device__ __forceinline__ uint2 quant_group8(const float (&x)[8], const RowQuant& p) {
  const float shift = (float)(p.zp + 128);
  uint32_t w[2] = {0u, 0u};
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float r = round_half_away(__fmul_rn(x[e], p.scale));
    w[e >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(__fadd_rn(r, shift), e & 3, w[e >> 2]);
  }
  return make_uint2(w[0] ^ 0x80808080u, w[1] ^ 0x80808080u);
}

// Wavefront-wide min / max with DPP lane permutations (no LDS traffic): after the four
// in-row steps every lane holds its 16-lane row's result; two row broadcasts bring the total to
// lane 63, which is read back as a scalar.
template <bool kIsMax>
__device__ __forceinline__ float wave_minmax(float v) {
#define W4_DPP_STEP(ctrl, row_mask)                                                          \
  {                                                                                          \
    const float o = __int_as_float(__builtin_amdgcn_update_dpp(                              \
        __float_as_int(v), __float_as_int(v), (ctrl), (row_mask), 0xf, false));              \
    v = kIsMax ? fmaxf(v, o) : fminf(v, o);                                                  \
  }
  W4_DPP_STEP(0xB1, 0xf)   // quad_perm [1,0,3,2]
  W4_DPP_STEP(0x4E, 0xf)   // quad_perm [2,3,0,1]
  W4_DPP_STEP(0x141, 0xf)  // row_half_mirror
  W4_DPP_STEP(0x140, 0xf)  // row_mirror
  W4_DPP_STEP(0x142, 0xa)  // row_bcast:15 into rows 1 and 3
  W4_DPP_STEP(0x143, 0xc)  // row_bcast:31 into rows 2 and 3
#undef W4_DPP_STEP
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// min and max of two values per lane across the wavefront, both chains interleaved so that each
// DPP read finds its register two issue slots after the write. The totals end up in lane 63.
__device__ __forceinline__ void wave_minmax_pair(float& lo, float& hi) {
  asm volatile(
      "s_nop 1\n\t"
      "v_min_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(lo), "+v"(hi));
}

// The same within every row of 16 lanes; all 16 lanes of a row end up with the row's totals.
__device__ __forceinline__ void row16_minmax_pair(float& lo, float& hi) {
  asm volatile(
      "s_nop 1\n\t"
      "v_min_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 0\n\t"
      "v_min_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(lo), "+v"(hi));
}

// Sum across the wavefront; the total ends up in lane 63. Same steps as the min/max pair.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  asm volatile(
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(v));
  return v;
}

// Sum within every row of 16 lanes; all 16 lanes of a row end up with the row's total.
__device__ __forceinline__ float row16_sum_all(float v) {
  asm volatile(
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1"
      : "+v"(v));
  return v;
}

}  // namespace w4
