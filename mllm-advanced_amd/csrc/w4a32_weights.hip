// Offline weight kernels: the 4-bit block-32 quantizer, the repack into the tiled device
// layout, its inverse, and the dequantizer. All integer/byte work, bit-exact by contract.
#include "w4a32_internal.h"

namespace w4 {

// ----------------------------------------------------------------------------------------
// f32 [N][K] -> offset-8 nibbles [N][K/2] + bf16 scales [N][K/32].
// Same arithmetic, in the same order, as the reference's scalar quantizer
// (mllm/Backends/Arm/Kernels/kai_linear.cpp:233-289): first element of largest magnitude,
// scale = it / -8, recip = scale ? 1/scale : 0, q = clamp(round_half_away(x * recip), -8, 7).
// One thread owns one (row, block): the sequential scan keeps the "first maximum wins" rule.
// ----------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void quant_rhs_kernel(const float* __restrict__ w, int N, int K,
                                                        uint8_t* __restrict__ u4,
                                                        uint16_t* __restrict__ scales, int rne) {
  const int nb = K / kBlockLen;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)N * nb) return;
  const int n = (int)(idx / nb);
  const int b = (int)(idx % nb);

  float v[kBlockLen];
  const float4* src = reinterpret_cast<const float4*>(w + (size_t)n * K + (size_t)b * kBlockLen);
#pragma unroll
  for (int i = 0; i < kBlockLen / 4; ++i) {
    const float4 t = src[i];
    v[4 * i + 0] = t.x;
    v[4 * i + 1] = t.y;
    v[4 * i + 2] = t.z;
    v[4 * i + 3] = t.w;
  }

  float best_abs = 0.0f, best = 0.0f;
#pragma unroll
  for (int i = 0; i < kBlockLen; ++i) {
    const float a = fabsf(v[i]);
    if (best_abs < a) {
      best_abs = a;
      best = v[i];
    }
  }
  const float scale = __fdiv_rn(best, -8.0f);  // exact unless it lands in the denormals
  const float recip = (scale != 0.0f) ? __fdiv_rn(1.0f, scale) : 0.0f;

  uint32_t bits = __float_as_uint(scale);
  if (rne) {
    if ((bits & 0x7fffffffu) > 0x7f800000u) {
      bits = (bits >> 16) | 0x0040u;
    } else {
      bits = (bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16;
    }
  } else {
    bits >>= 16;
  }
  scales[(size_t)n * nb + b] = (uint16_t)bits;

  uint32_t out[4] = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int i = 0; i < kBlockLen; ++i) {
    const float r = roundf(__fmul_rn(v[i], recip));  // f32 product, then half away from zero
    int q = (int)fminf(fmaxf(r, -8.0f), 7.0f);
    out[i >> 3] |= (uint32_t)(q + 8) << (4 * (i & 7));  // even k -> low nibble of byte k/2
  }
  uint4* dst = reinterpret_cast<uint4*>(u4 + (size_t)n * (K / 2) + (size_t)b * 16);
  *dst = make_uint4(out[0], out[1], out[2], out[3]);
}

// Row-major dword (nibble p = k0 + p, offset-8) <-> tile dword (see w4a32_layout.h).
__device__ __forceinline__ uint32_t to_tile_dword(uint32_t src) {
  uint32_t dst = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t t = ((src >> (4 * e)) & 0xFu) ^ 8u;  // two's complement of q = u4 - 8
    dst |= t << (4 * nibble_pos(e));
  }
  return dst;
}

__device__ __forceinline__ uint32_t from_tile_dword(uint32_t tile) {
  uint32_t src = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t u = ((tile >> (4 * nibble_pos(e))) & 0xFu) ^ 8u;
    src |= u << (4 * e);
  }
  return src;
}

// One wavefront per tile: lane l writes its own 16 bytes and one of the 64 scales.
__global__ __launch_bounds__(64) void repack_kernel(const uint8_t* __restrict__ u4,
                                                    const uint16_t* __restrict__ scales, int N,
                                                    int K, int KC, uint8_t* __restrict__ packed) {
  const int tile = blockIdx.x;
  const int nt = tile / KC, kc = tile % KC;
  const int l = threadIdx.x, g = l >> 4, j = l & 15;
  const int nb = K / kBlockLen;
  const int n = kTileRows * nt + j;

  uint32_t o[4];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int k0 = kTileK * kc + kBlockLen * d + 8 * g;
    uint32_t src = 0x88888888u;  // q = 0 in padding
    if (n < N && k0 < K) {
      src = *reinterpret_cast<const uint32_t*>(u4 + (size_t)n * (K / 2) + k0 / 2);
    }
    o[d] = to_tile_dword(src);
  }
  uint8_t* base = packed + (size_t)tile * kTileBytes;
  *reinterpret_cast<uint4*>(base + 16 * l) = make_uint4(o[0], o[1], o[2], o[3]);

  const int sj = l >> 2, sd = l & 3;
  const int sn = kTileRows * nt + sj, sb = 4 * kc + sd;
  uint16_t s = 0;
  if (sn < N && sb < nb) s = scales[(size_t)sn * nb + sb];
  *reinterpret_cast<uint16_t*>(base + kTileQBytes + 2 * l) = s;
}

// E_n such that (largest |scale| of the row) * 2^-E_n lies in [2^11, 2^12); 0 for an all-zero row.
// mag = bf16 bits of that scale without the sign. bf16 subnormals count as exponent -126.
__device__ __forceinline__ int row_exponent(uint32_t mag) {
  if (mag == 0) return 0;
  int e = (int)(mag >> 7) - 127;
  if ((mag >> 7) == 0) e = -126;
  return e - 11;
}

// Per-row sum_b f32(scale_b) * (float)(sum_{k in b} q) in block order, the bias plane, and the
// power of two that normalises the row's scales for the f16 copy.
__global__ __launch_bounds__(256) void rsum_bias_kernel(const uint8_t* __restrict__ u4,
                                                        const uint16_t* __restrict__ scales,
                                                        const float* __restrict__ bias, int N,
                                                        int K, int Np, float* __restrict__ rsum,
                                                        float* __restrict__ bias_out,
                                                        float* __restrict__ rowmul) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= Np) return;
  float r = 0.0f, bv = 0.0f;
  uint32_t max_mag = 0;  // largest |scale| of the row, as bf16 bits without the sign
  if (n < N) {
    const int nb = K / kBlockLen;
    const uint4* row = reinterpret_cast<const uint4*>(u4 + (size_t)n * (K / 2));
    for (int b = 0; b < nb; ++b) {
      const uint4 v = row[b];
      const uint32_t wv[4] = {v.x, v.y, v.z, v.w};
      int s = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // sum of the 8 nibbles of a dword
        uint32_t t = (wv[i] & 0x0F0F0F0Fu) + ((wv[i] >> 4) & 0x0F0F0F0Fu);
        t = (t & 0x00FF00FFu) + ((t >> 8) & 0x00FF00FFu);
        s += (int)((t & 0xFFFFu) + (t >> 16));
      }
      s -= 8 * kBlockLen;
      const uint32_t sbits = scales[(size_t)n * nb + b];
      r = __fadd_rn(r, __fmul_rn((float)s, bf16_bits_to_f32(sbits)));
      const uint32_t mag = sbits & 0x7FFFu;
      if (mag < 0x7F80u && mag > max_mag) max_mag = mag;  // ignore inf/nan scales
    }
    if (bias) bv = bias[n];
  }
  rsum[n] = r;
  bias_out[n] = bv;
  rowmul[n] = ldexpf(1.0f, row_exponent(max_mag));
}

// f16 copy of the block scales, each row divided by its rowmul (a power of two).
__global__ __launch_bounds__(64) void hscale_kernel(const uint16_t* __restrict__ scales, int N,
                                                    int K, int KC, const float* __restrict__ rowmul,
                                                    _Float16* __restrict__ hscale) {
  const int tile = blockIdx.x;
  const int nt = tile / KC, kc = tile % KC;
  const int l = threadIdx.x;
  const int nb = K / kBlockLen;
  const int sn = kTileRows * nt + (l >> 2), sb = 4 * kc + (l & 3);
  float v = 0.0f;
  if (sn < N && sb < nb) {
    int e;
    (void)frexpf(rowmul[sn], &e);  // rowmul = 2^(e-1)
    v = ldexpf(bf16_bits_to_f32(scales[(size_t)sn * nb + sb]), -(e - 1));
  }
  hscale[(size_t)tile * 64 + l] = (_Float16)v;
}

__global__ __launch_bounds__(64) void unpack_kernel(const uint8_t* __restrict__ packed, int N,
                                                    int K, int KC, uint8_t* __restrict__ u4,
                                                    uint16_t* __restrict__ scales) {
  const int tile = blockIdx.x;
  const int nt = tile / KC, kc = tile % KC;
  const int l = threadIdx.x, g = l >> 4, j = l & 15;
  const int nb = K / kBlockLen;
  const int n = kTileRows * nt + j;
  const uint8_t* base = packed + (size_t)tile * kTileBytes;
  const uint4 v = *reinterpret_cast<const uint4*>(base + 16 * l);
  const uint32_t wv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int k0 = kTileK * kc + kBlockLen * d + 8 * g;
    if (n < N && k0 < K) {
      *reinterpret_cast<uint32_t*>(u4 + (size_t)n * (K / 2) + k0 / 2) = from_tile_dword(wv[d]);
    }
  }
  const int sj = l >> 2, sd = l & 3;
  const int sn = kTileRows * nt + sj, sb = 4 * kc + sd;
  if (sn < N && sb < nb) {
    scales[(size_t)sn * nb + sb] = *reinterpret_cast<const uint16_t*>(base + kTileQBytes + 2 * l);
  }
}

// [parity unpinned] The blob the reference's Arm quantizer stores (output of
// kai_run_rhs_pack_nxk_qsi4c32p_qsu4c32s1s0, called at kai_linear.cpp:331-344) back to the native
// arrays. KleidiAI is not part of the reference tree; the layout is restated from its published
// packing loop: rows in groups of nr; per group and 32-block nr*16 data bytes, where byte i belongs
// to segment i / (nr*seg), row (i / seg) % nr, position t = i % seg (seg = kr/sr), low nibble =
// weight k = seg*segment + t of the block, high nibble = k + 16, the byte XORed with 0x88; then nr
// bf16 scales; after the group's blocks nr f32 row sums (not used here) and nr f32 biases.
// One thread per (row, block).
__global__ __launch_bounds__(256) void unpack_kai_kernel(const uint8_t* __restrict__ blob, int N,
                                                         int K, int nr, int seg,
                                                         uint8_t* __restrict__ u4,
                                                         uint16_t* __restrict__ scales,
                                                         float* __restrict__ bias) {
  const int nb = K / kBlockLen;
  const long id = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= (long)N * nb) return;
  const int n = (int)(id / nb), b = (int)(id % nb);
  const int grp = n / nr, r = n % nr;
  const size_t group_bytes = (size_t)nr * ((size_t)nb * 18 + 8);
  const uint8_t* gbase = blob + (size_t)grp * group_bytes;
  const uint8_t* data = gbase + (size_t)b * nr * 18;
  uint8_t lo[16], hi[16];  // u4 at k = 0..15 and 16..31 of the block
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const int s = k / seg, t = k % seg;
    const uint8_t v = data[(s * nr + r) * seg + t] ^ 0x88;
    lo[k] = v & 0xF;
    hi[k] = v >> 4;
  }
  uint8_t* dst = u4 + (size_t)n * (K / 2) + 16 * b;  // native: byte k/2, low nibble = even k
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    dst[i] = (uint8_t)(lo[2 * i] | (lo[2 * i + 1] << 4));
    dst[8 + i] = (uint8_t)(hi[2 * i] | (hi[2 * i + 1] << 4));
  }
  const uint8_t* sp = data + nr * 16 + 2 * r;
  scales[(size_t)n * nb + b] = (uint16_t)(sp[0] | (sp[1] << 8));
  if (b == 0 && bias) {
    const uint8_t* bp = gbase + (size_t)nb * nr * 18 + 4 * nr + 4 * r;
    const uint32_t bits = bp[0] | (bp[1] << 8) | (bp[2] << 16) | ((uint32_t)bp[3] << 24);
    bias[n] = __uint_as_float(bits);
  }
}

__global__ __launch_bounds__(256) void copy_bias_kernel(const float* __restrict__ src, int N,
                                                        float* __restrict__ dst) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n < N) dst[n] = src[n];
}

// tile -> f32 [N][K]: (float)q * f32(scale); one exact product per weight.
__global__ __launch_bounds__(64) void dequant_kernel(const uint8_t* __restrict__ packed, int N,
                                                     int K, int KC, float* __restrict__ out) {
  const int tile = blockIdx.x;
  const int nt = tile / KC, kc = tile % KC;
  const int l = threadIdx.x, g = l >> 4, j = l & 15;
  const int n = kTileRows * nt + j;
  if (n >= N) return;
  const uint8_t* base = packed + (size_t)tile * kTileBytes;
  const uint4 v = *reinterpret_cast<const uint4*>(base + 16 * l);
  const uint2 sc = *reinterpret_cast<const uint2*>(base + kTileQBytes + 8 * j);
  const uint32_t wv[4] = {v.x, v.y, v.z, v.w};
  const uint32_t sb[4] = {sc.x & 0xFFFFu, sc.x >> 16, sc.y & 0xFFFFu, sc.y >> 16};
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int k0 = kTileK * kc + kBlockLen * d + 8 * g;
    if (k0 >= K) continue;
    const float s = bf16_bits_to_f32(sb[d]);
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int q = ((int)(wv[d] << (28 - 4 * nibble_pos(e)))) >> 28;  // sign-extend the nibble
      f[e] = __fmul_rn((float)q, s);
    }
    float4* dst = reinterpret_cast<float4*>(out + (size_t)n * K + k0);
    dst[0] = make_float4(f[0], f[1], f[2], f[3]);
    dst[1] = make_float4(f[4], f[5], f[6], f[7]);
  }
}

// ----------------------------------------------------------------------------------------

hipError_t launch_quant_rhs(const float* w, int N, int K, uint8_t* u4, uint16_t* scales, int rne,
                            hipStream_t s) {
  const long total = (long)N * (K / kBlockLen);
  const unsigned grid = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(quant_rhs_kernel, dim3(grid), dim3(256), 0, s, w, N, K, u4, scales, rne);
  return hipGetLastError();
}

hipError_t launch_repack(const uint8_t* u4, const uint16_t* scales, const float* bias, int N, int K,
                         uint8_t* packed, hipStream_t s) {
  const WeightGeom g = weight_geom(N, K);
  hipLaunchKernelGGL(repack_kernel, dim3(g.NT * g.KC), dim3(64), 0, s, u4, scales, N, K, g.KC,
                     packed);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(rsum_bias_kernel, dim3((g.Np + 255) / 256), dim3(256), 0, s, u4, scales, bias,
                     N, K, g.Np, reinterpret_cast<float*>(packed + g.rsum_off),
                     reinterpret_cast<float*>(packed + g.bias_off),
                     reinterpret_cast<float*>(packed + g.rowmul_off));
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(hscale_kernel, dim3(g.NT * g.KC), dim3(64), 0, s, scales, N, K, g.KC,
                     reinterpret_cast<const float*>(packed + g.rowmul_off),
                     reinterpret_cast<_Float16*>(packed + g.hscale_off));
  return hipGetLastError();
}

hipError_t launch_unpack(const uint8_t* packed, int N, int K, uint8_t* u4, uint16_t* scales,
                         float* bias, hipStream_t s) {
  const WeightGeom g = weight_geom(N, K);
  hipLaunchKernelGGL(unpack_kernel, dim3(g.NT * g.KC), dim3(64), 0, s, packed, N, K, g.KC, u4,
                     scales);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || !bias) return e;
  hipLaunchKernelGGL(copy_bias_kernel, dim3((N + 255) / 256), dim3(256), 0, s,
                     reinterpret_cast<const float*>(packed + g.bias_off), N, bias);
  return hipGetLastError();
}

hipError_t launch_unpack_kai(const uint8_t* blob, int N, int K, int nr, int kr, int sr, uint8_t* u4,
                             uint16_t* scales, float* bias, hipStream_t s) {
  const long items = (long)N * (K / kBlockLen);
  hipLaunchKernelGGL(unpack_kai_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, s, blob, N,
                     K, nr, kr / sr, u4, scales, bias);
  return hipGetLastError();
}

hipError_t launch_dequant(const uint8_t* packed, int N, int K, float* out, hipStream_t s) {
  const WeightGeom g = weight_geom(N, K);
  hipLaunchKernelGGL(dequant_kernel, dim3(g.NT * g.KC), dim3(64), 0, s, packed, N, K, g.KC, out);
  return hipGetLastError();
}

}  // namespace w4
