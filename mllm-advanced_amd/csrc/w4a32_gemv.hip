// Decode product (M = 1..8): y[M][N] from int8 activation rows and the tiled 4-bit weights.
//
// HBM-bound: per output row the kernel must stream K/2 bytes of nibbles and K/16 bytes of
// scales once; everything else (activations, rsum, bias) is a few KB that live in L2/LDS.
//
// Work split: one workgroup per 16-row weight tile row (nt); its W wavefronts take the
// 128-k chunks round-robin, so a workgroup streams one contiguous KC*1152-byte run.
// A wavefront's 128-bit-per-lane load is one whole 1 KiB tile. The next chunk is requested
// before the current one is consumed. Activations are staged once per workgroup into LDS
// (after the first weight loads are in flight) and read back as 64-bit broadcasts.
//
// Arithmetic per 8 weights (one dword): two mask ops give int8 vectors of 16*q, two
// v_dot4_i32_i8 give 16 * sum a_q*q exactly, one cvt + one fma apply the block scale in f32.
// The 1/16 and the activation offset (off * rsum[n]) are folded in once per output.
#include "w4a32_internal.h"

namespace w4 {

template <int M>
__global__ __launch_bounds__(1024) void gemv_dot4_kernel(
    float* __restrict__ y, const int8_t* __restrict__ aq, const float* __restrict__ recip,
    const int32_t* __restrict__ negzp, const uint8_t* __restrict__ packed, int N, int K, int KC,
    const float* __restrict__ rsum, const float* __restrict__ bias) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int Kp = KC * kTileK;
  int8_t* s_a = reinterpret_cast<int8_t*>(smem);                  // [M][Kp]
  float* s_red = reinterpret_cast<float*>(smem + (size_t)M * Kp); // [W][M][16]

  const int nt = blockIdx.x;
  const int W = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 4, j = lane & 15;

  const uint8_t* tiles = packed + (size_t)nt * KC * kTileBytes;

  // First chunk of this wavefront: in flight while the activations are staged.
  int kc = wave;
  uint4 wq = make_uint4(0, 0, 0, 0);
  uint2 sc = make_uint2(0, 0);
  if (kc < KC) {
    wq = *reinterpret_cast<const uint4*>(tiles + (size_t)kc * kTileBytes + 16 * lane);
    sc = *reinterpret_cast<const uint2*>(tiles + (size_t)kc * kTileBytes + kTileQBytes + 8 * j);
  }

  // Stage a_q into LDS, 16 bytes per thread per step; k >= K (tile padding) reads as 0.
  const int vec_per_row = Kp / 16;
  for (int v = threadIdx.x; v < M * vec_per_row; v += blockDim.x) {
    const int m = v / vec_per_row, c = v % vec_per_row;
    uint4 val = make_uint4(0, 0, 0, 0);
    if (16 * c < K) val = *reinterpret_cast<const uint4*>(aq + (size_t)m * K + 16 * c);
    *reinterpret_cast<uint4*>(s_a + (size_t)m * Kp + 16 * c) = val;
  }
  __syncthreads();

  float acc[M];
#pragma unroll
  for (int m = 0; m < M; ++m) acc[m] = 0.0f;

  while (kc < KC) {
    const int kn = kc + W;
    uint4 wq_n = make_uint4(0, 0, 0, 0);
    uint2 sc_n = make_uint2(0, 0);
    if (kn < KC) {
      wq_n = *reinterpret_cast<const uint4*>(tiles + (size_t)kn * kTileBytes + 16 * lane);
      sc_n = *reinterpret_cast<const uint2*>(tiles + (size_t)kn * kTileBytes + kTileQBytes + 8 * j);
    }

    const uint32_t wv[4] = {wq.x, wq.y, wq.z, wq.w};
    const float sv[4] = {__uint_as_float(sc.x << 16), __uint_as_float(sc.x & 0xFFFF0000u),
                         __uint_as_float(sc.y << 16), __uint_as_float(sc.y & 0xFFFF0000u)};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int lo = (int)((wv[d] << 4) & 0xF0F0F0F0u);  // 16*q at k offsets 0..3
      const int hi = (int)(wv[d] & 0xF0F0F0F0u);         // 16*q at k offsets 4..7
      const int8_t* a_base = s_a + kTileK * kc + kBlockLen * d + 8 * g;
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const int2 a = *reinterpret_cast<const int2*>(a_base + (size_t)m * Kp);
        int dot = __builtin_amdgcn_sdot4(a.x, lo, 0, false);
        dot = __builtin_amdgcn_sdot4(a.y, hi, dot, false);
        acc[m] = __fmaf_rn((float)dot, sv[d], acc[m]);
      }
    }
    kc = kn;
    wq = wq_n;
    sc = sc_n;
  }

  // Sum the four k-groups of a row (lanes j, j+16, j+32, j+48), then the wavefronts.
#pragma unroll
  for (int m = 0; m < M; ++m) {
    acc[m] += __shfl_xor(acc[m], 16, 64);
    acc[m] += __shfl_xor(acc[m], 32, 64);
  }
  if (g == 0) {
#pragma unroll
    for (int m = 0; m < M; ++m) s_red[(wave * M + m) * 16 + j] = acc[m];
  }
  __syncthreads();

  // 16*M outputs; a workgroup may have as few as 64 threads, so stride over them.
  for (int o = threadIdx.x; o < 16 * M; o += blockDim.x) {
    const int m = o >> 4, jj = o & 15;
    const int n = kTileRows * nt + jj;
    if (n < N) {
      float s = 0.0f;
      for (int w = 0; w < W; ++w) s += s_red[(w * M + m) * 16 + jj];
      float v = __fmaf_rn((float)negzp[m], rsum[n], s * 0.0625f);
      v = __fmaf_rn(v, recip[m], bias[n]);
      v = fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
      y[(size_t)m * N + n] = v;
    }
  }
}

static int pick_waves(int KC) { return KC < 16 ? KC : 16; }

template <int M>
static hipError_t launch_gemv_m(float* y, const uint8_t* ws, const uint8_t* packed, int K, int N,
                                hipStream_t s) {
  const WeightGeom g = weight_geom(N, K);
  const WsGeom w = ws_geom(M, K);
  const int W = pick_waves(g.KC);
  const size_t lds = (size_t)M * g.Kp + (size_t)W * M * 16 * sizeof(float);
  auto kern = gemv_dot4_kernel<M>;
  if (lds > 64 * 1024) {
    static bool raised = false;  // one attribute call per instantiation is enough
    if (!raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (e != hipSuccess) return e;
      raised = true;
    }
  }
  hipLaunchKernelGGL(kern, dim3(g.NT), dim3(64 * W), lds, s, y,
                     reinterpret_cast<const int8_t*>(ws + w.aq_off),
                     reinterpret_cast<const float*>(ws + w.scale_off),
                     reinterpret_cast<const int32_t*>(ws + w.off_off), packed, N, K, g.KC,
                     reinterpret_cast<const float*>(packed + g.rsum_off),
                     reinterpret_cast<const float*>(packed + g.bias_off));
  return hipGetLastError();
}

hipError_t launch_gemv(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                       hipStream_t s) {
  switch (M) {
    case 1: return launch_gemv_m<1>(y, ws, packed, K, N, s);
    case 2: return launch_gemv_m<2>(y, ws, packed, K, N, s);
    case 3: return launch_gemv_m<3>(y, ws, packed, K, N, s);
    case 4: return launch_gemv_m<4>(y, ws, packed, K, N, s);
    case 5: return launch_gemv_m<5>(y, ws, packed, K, N, s);
    case 6: return launch_gemv_m<6>(y, ws, packed, K, N, s);
    case 7: return launch_gemv_m<7>(y, ws, packed, K, N, s);
    case 8: return launch_gemv_m<8>(y, ws, packed, K, N, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace w4
