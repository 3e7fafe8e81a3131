// Decode product (M = 1..8): y[M][N] from f32 or already-quantised activation rows and the
// tiled 4-bit weights.
//
// HBM-bound: per output row the kernel must stream K/2 bytes of nibbles and K/16 bytes of
// scales once; everything else (activations, rsum, bias) is a few KB that live in L2/LDS.
//
// Work split: one workgroup per 16-row weight tile row (nt); its W wavefronts take the
// 128-k chunks round-robin, so a workgroup streams one contiguous KC*1152-byte run.
// A wavefront's 128-bit-per-lane load is one whole 1 KiB tile. The first chunk is requested
// before anything else happens, the next one before the current one is consumed.
//
// For very wide layers (N >= 32768, e.g. a vocabulary projection) gemv_wide_kernel gives every
// WAVEFRONT whole tile rows instead: it keeps four chunk loads in flight, needs no cross-wavefront
// reduction and therefore no barrier after the activations are staged - that is the shape where
// the kernel is genuinely bandwidth-bound.
//
// Two entry kernels share the loop:
//   gemv_q_kernel      activations already quantised (workspace of w4a32_quant_lhs)
//   gemv_fused_kernel  quantises the f32 rows itself: every workgroup recomputes the row
//                      min/max (a few KB from L2, DPP reductions) and quantises into its own
//                      LDS copy with the same arithmetic as the standalone kernel. This removes
//                      one kernel launch per Linear, which at decode sizes costs more than the
//                      product itself.
//
// Arithmetic per 8 weights (one dword): two mask ops give int8 vectors of 16*q, two
// v_dot4_i32_i8 give 16 * sum a_q*q exactly, one cvt + one fma apply the block scale in f32.
// The 1/16 and the activation offset (off * rsum[n]) are folded in once per output.
//
// From three rows on (kDecodeMfmaMinM) the dot products of a scale block come from ONE
// v_mfma_i32_16x16x32_i8 instead of 2*M v_dot4: the tile dword of all 64 lanes, expanded by the
// same two mask ops, is its B operand (column = lane % 16, k-slice = lane / 16), the A operand is
// 8 bytes of activation row lane % 16 (rows past M repeat the last one; their results are not
// used). Lane (g, j) then holds the exact block sums of rows 4g..4g+3 for column j, already
// summed over the four k-groups; cvt + fma apply the block scale as before, so every output is
// the same f32 expression in the same order as on the dot4 path. The instruction count per chunk
// no longer grows with M (M = 8: 130 -> 45 per wavefront).
#include <algorithm>

#include "w4a32_internal.h"
#include "w4a32_quant_math.h"

namespace w4 {

typedef int v4i_t __attribute__((ext_vector_type(4)));
constexpr int kDecodeMfmaMinM = 3;
constexpr bool decode_mfma(int M) { return M >= kDecodeMfmaMinM; }
// accumulators per lane: one per row (a partial over this lane's k-group) or, on the MFMA path,
// rows 4g..4g+3 of column j
constexpr int decode_acc(int M) { return decode_mfma(M) ? 4 : M; }

// One scale block (tile dword wv, scale sv) against the M int8 rows at a_base (+ m * Kp, the row stride of
// the caller's layout); a_base already points at this lane's k-group.
template <int M>
__device__ __forceinline__ void block_products(uint32_t wv, float sv, const int8_t* a_base, int Kp,
                                               int j, float (&acc)[decode_acc(M)]) {
  const uint32_t lo = (wv << 4) & 0xF0F0F0F0u;  // 16*q at k offsets 0..3
  const uint32_t hi = wv & 0xF0F0F0F0u;         // 16*q at k offsets 4..7
  if constexpr (decode_mfma(M)) {
    const long b64 = (long)(((unsigned long)hi << 32) | lo);
    const long a64 = *reinterpret_cast<const long*>(a_base + (size_t)(j < M ? j : M - 1) * Kp);
    v4i_t c = {0, 0, 0, 0};
    c = __builtin_amdgcn_mfma_i32_16x16x32_i8(a64, b64, c, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] = __fmaf_rn((float)c[r], sv, acc[r]);
  } else {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const int2 a = *reinterpret_cast<const int2*>(a_base + (size_t)m * Kp);
      int dot = __builtin_amdgcn_sdot4(a.x, (int)lo, 0, false);
      dot = __builtin_amdgcn_sdot4(a.y, (int)hi, dot, false);
      acc[m] = __fmaf_rn((float)dot, sv, acc[m]);
    }
  }
}

// The sums of a wavefront, complete over its k-groups, to s_dst[m * 16 + j].
template <int M>
__device__ __forceinline__ void store_row_sums(float (&acc)[decode_acc(M)], float* s_dst, int lane) {
  const int g = lane >> 4, j = lane & 15;
  if constexpr (decode_mfma(M)) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = 4 * g + r;
      if (m < M) s_dst[m * 16 + j] = acc[r];
    }
  } else {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float v = acc[m];
      v += __shfl_xor(v, 16, 64);
      v += __shfl_xor(v, 32, 64);
      if (lane < 16) s_dst[m * 16 + lane] = v;
    }
  }
}

// Streams this wavefront's chunks of tile row `tiles` against the int8 rows in LDS and leaves
// the per-(m, j) sums over the whole workgroup in s_red[m*16 + j] order via a final reduction.
template <int M>
__device__ __forceinline__ void gemv_accumulate(const uint8_t* __restrict__ tiles, int KC, int Kp,
                                                const int8_t* s_a, uint4 wq, uint2 sc, int kc,
                                                int W, int lane, float (&acc)[decode_acc(M)]) {
  const int g = lane >> 4, j = lane & 15;
#pragma unroll
  for (int m = 0; m < decode_acc(M); ++m) acc[m] = 0.0f;

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
      block_products<M>(wv[d], sv[d], s_a + kTileK * kc + kBlockLen * d + 8 * g, Kp, j, acc);
    }
    kc = kn;
    wq = wq_n;
    sc = sc_n;
  }
}

constexpr int kMaxWaves = 16;  // wavefronts per workgroup, at most

// Cross-wavefront sum and the output transform
//   y = (sum/16 + off * rsum[n]) * lhs_scale + bias[n], clamped to the finite f32 range.
// When the workgroup has at least 16*M threads, thread o owns output o and already holds
// rsum/bias of its column (rs, bs: requested at kernel start); smaller workgroups (K < 128*M/4)
// stride over the outputs and fetch them here.
template <int M>
__device__ __forceinline__ void gemv_finish(float* __restrict__ y, int N, int nt, int W,
                                            float (&acc)[decode_acc(M)], float* s_red,
                                            const float (&recip_m)[M], const int (&negzp_m)[M],
                                            const float* __restrict__ rsum,
                                            const float* __restrict__ bias, float rs, float bs) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  store_row_sums<M>(acc, s_red + wave * M * 16, lane);
  __syncthreads();
  const bool prefetched = blockDim.x >= 16 * M;
  for (int o = threadIdx.x; o < 16 * M; o += blockDim.x) {
    const int m = o >> 4, jj = o & 15;
    const int n = kTileRows * nt + jj;
    if (n < N) {
      // All kMaxWaves reads are issued before the first add (a loop over W would wait for each
      // LDS read in turn); wavefronts past W re-read the last one and add 0.
      float part[kMaxWaves];
#pragma unroll
      for (int w = 0; w < kMaxWaves; ++w) part[w] = s_red[((w < W ? w : W - 1) * M + m) * 16 + jj];
      float s = 0.0f;
#pragma unroll
      for (int w = 0; w < kMaxWaves; ++w) s += w < W ? part[w] : 0.0f;
      float rcp = 0.0f;
      int off = 0;
#pragma unroll
      for (int mm = 0; mm < M; ++mm) {  // compile-time indices keep the arrays in registers
        if (mm == m) {
          rcp = recip_m[mm];
          off = negzp_m[mm];
        }
      }
      const float rsn = prefetched ? rs : rsum[n];
      const float bsn = prefetched ? bs : bias[n];
      float v = __fmaf_rn((float)off, rsn, s * 0.0625f);
      v = __fmaf_rn(v, rcp, bsn);
      v = fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
      y[(size_t)m * N + n] = v;
    }
  }
}

template <int M>
__global__ __launch_bounds__(1024) void gemv_q_kernel(
    float* __restrict__ y, const int8_t* __restrict__ aq, const float* __restrict__ recip,
    const int32_t* __restrict__ negzp, const uint8_t* __restrict__ packed, int N, int K, int KC,
    const float* __restrict__ rsum, const float* __restrict__ bias) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int Kp = KC * kTileK;
  int8_t* s_a = reinterpret_cast<int8_t*>(smem);                    // [M][Kp]
  float* s_red = reinterpret_cast<float*>(smem + (size_t)M * Kp);   // [W][M][16]
  float* s_par = s_red + (blockDim.x >> 6) * M * 16;                // recip[M], negzp[M]

  const int nt = blockIdx.x;
  const int W = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint8_t* tiles = packed + (size_t)nt * KC * kTileBytes;

  // First chunk of this wavefront: in flight while the activations are staged.
  uint4 wq = make_uint4(0, 0, 0, 0);
  uint2 sc = make_uint2(0, 0);
  if (wave < KC) {
    wq = *reinterpret_cast<const uint4*>(tiles + (size_t)wave * kTileBytes + 16 * lane);
    sc = *reinterpret_cast<const uint2*>(tiles + (size_t)wave * kTileBytes + kTileQBytes +
                                         8 * (lane & 15));
  }
  // Output-transform operands, requested now so the epilogue does not wait on memory.
  float rs = 0.0f, bs = 0.0f;
  {
    const int n = kTileRows * nt + (threadIdx.x & 15);
    if (threadIdx.x < 16 * M && n < N) {
      rs = rsum[n];
      bs = bias[n];
    }
  }
  if (threadIdx.x < M) {
    s_par[threadIdx.x] = recip[threadIdx.x];
    reinterpret_cast<int*>(s_par)[M + threadIdx.x] = negzp[threadIdx.x];
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

  float acc[decode_acc(M)];
  gemv_accumulate<M>(tiles, KC, Kp, s_a, wq, sc, wave, W, lane, acc);
  float recip_m[M];
  int negzp_m[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    recip_m[m] = s_par[m];
    negzp_m[m] = reinterpret_cast<const int*>(s_par)[M + m];
  }
  gemv_finish<M>(y, N, nt, W, acc, s_red, recip_m, negzp_m, rsum, bias, rs, bs);
}

// Up to kMaxGroup Linears that share their activation rows (and therefore K), run by one launch:
// workgroup b serves tile row b - first[i] of Linear i, where first[] are running sums of tile rows.
constexpr int kMaxGroup = 4;
struct RowPrologue {
  const float* delta;   // optional: added to x before anything else
  float* sum_out;       // optional: receives x + delta (must not alias x)
  const float* norm_w;  // RMSNorm weight [K]
  float eps;
  int delta_parts;      // gemv_wide_kernel: delta is the sum of that many rows, K floats apart (0 or 1: one row)
  // gemv_wide_kernel at M = 1: when given, wavefront w of the launch also leaves the largest of the outputs it
  // stored and its column (the first such column; -inf and 0x7fffffff when it stored none) in amax_val[w],
  // amax_idx[w], for a greedy sampler that then looks at wide_partials() pairs instead of N outputs
  float* amax_val;
  int* amax_idx;
};
struct GroupArgs {
  const uint8_t* packed[kMaxGroup];
  float* y[kMaxGroup];
  int N[kMaxGroup];
  int first[kMaxGroup + 1];  // first[i] = tile rows of Linears 0..i-1; first[count] = grid size
  int count;
  int in_parts;  // > 1: the input row (the delta row with a norm in front) is the sum of that many rows, K floats apart
  int pair_both; // kPair only: store both Linears' outputs (to y[0] and y[1]) instead of silu(y0) * y1
};

// Whole op in one launch: x f32 [M][K] (row stride ldx) -> y.
//
// A workgroup of W wavefronts owns one tile row. Wavefront w holds its chunks w, w + W, ... (kCPW
// of them, covering KC <= kCPW * W); all kCPW loads are requested at kernel start. Each thread owns kFusedR groups of 8 activations per row (covering
// K <= 8 * kFusedR * blockDim.x), kept in registers from the min/max pass to the quantise pass.
// kGrouped = false: a single Linear, the group table is not consulted.
//
// Nearly every instruction here is executed once per wavefront and depends on the one before, so
// the kernel's duration at decode sizes is its instruction count times the issue latency: the
// reductions use one DPP instruction per step and the quantiser four VALU instructions per value.
//
// kNorm: the row is first completed and normalised, as the decoder does between its blocks:
//   x <- x + delta (when delta is given; workgroup 0 also stores the sum to sum_out),
//   x <- x * (norm_w * 1/sqrt(mean(x^2) + eps))       (the RMSNorm kernel's arithmetic)
// kPair: exactly two Linears of the same N (gate, up): a workgroup multiplies tile row nt of both
//   and stores silu(y0) * y1 to y[0] - or, with ga.pair_both, each output to its own y: two Linears of equal
//   N on one row then take half the workgroups of the grouped form, each with twice the weight loads in
//   flight (gate,up at K = 1536: 6.1 against 6.4 us).
template <int M, int kFusedR, bool kGrouped, int kCPW, bool kNorm, bool kPair, int kInParts = 1>
__global__ __launch_bounds__(M == 1 ? 1024 : 512) void gemv_fused_kernel(
    const float* __restrict__ x, int ldx, unsigned kw, const uint8_t* packed0, unsigned long long firsts,
    const float* pro_delta, const float* pro_norm_w, const uint8_t* packed1,
    const uint8_t* packed2,  // 16 dwords: preloaded
    float pro_eps, float* pro_sum_out, const GroupArgs ga) {
  // The leading arguments (everything the first loads need: the row, the weights of up to three Linears and the
  // tile rows at which one Linear ends and the next begins) are preloaded into SGPRs by the dispatcher, so the
  // first loads go out without waiting for the argument segment; a read of that segment takes about half a
  // microsecond, which is why nothing that is needed before the epilogue lives there (with the group's table
  // read from it, a grouped launch cost 0.33 us more than a single Linear of the same size).
  //   kw     = K | wavefronts << 16 | Linears << 24
  //   firsts = first[1] | first[2] << 16 | first[3] << 32 | first[4] << 48 (tile rows, see GroupArgs)
  extern __shared__ __align__(16) uint8_t smem[];
  constexpr int kSets = kPair ? 2 : 1;  // weight matrices a workgroup multiplies
  const int K = (int)(kw & 0xFFFFu), W = (int)((kw >> 16) & 31u);
  const int KC = (K + kTileK - 1) / kTileK;
  const uint8_t* packed = packed0;
  int nt_first = 0, gi = 0;
  int NT = (int)(firsts & 0xFFFFu);
  if (kGrouped) {
    // Which Linear this workgroup belongs to: from preloaded registers only. (A fourth Linear's weights come
    // from the table.)
    const int count = (int)(kw >> 24);
    const int f1 = (int)(firsts & 0xFFFFu), f2 = (int)((firsts >> 16) & 0xFFFFu),
              f3 = (int)((firsts >> 32) & 0xFFFFu), f4 = (int)(firsts >> 48);
    const int b = (int)blockIdx.x;
    if (count > 1 && b >= f1) {
      packed = packed1;
      nt_first = f1;
      NT = f2 - f1;
      gi = 1;
    }
    if (count > 2 && b >= f2) {
      packed = packed2;
      nt_first = f2;
      NT = f3 - f2;
      gi = 2;
    }
    if (count > 3 && b >= f3) {
      packed = ga.packed[3];
      nt_first = f3;
      NT = f4 - f3;
      gi = 3;
    }
  }
  // Output pointer and width of this workgroup's Linear: read from the argument segment now, used in the epilogue
  float* y = ga.y[0];
  int N = ga.N[0];
  if (kGrouped) {
#pragma unroll
    for (int i = 1; i < kMaxGroup; ++i) {
      if (gi == i) {
        y = ga.y[i];
        N = ga.N[i];
      }
    }
  }
  const float* rsum = reinterpret_cast<const float*>(packed + (size_t)NT * KC * kTileBytes);
  const int Kp = KC * kTileK;
  const int nthreads = 64 * W;  // the workgroup size, without a read of the hidden launch arguments
  int8_t* s_a = reinterpret_cast<int8_t*>(smem);                          // [M][Kp]
  float* s_red = reinterpret_cast<float*>(smem + (size_t)M * Kp);         // [W][kSets][M][16]
  float2* s_mm = reinterpret_cast<float2*>(s_red + W * kSets * M * 16);   // [W][M] (min, max)
  float* s_ss = reinterpret_cast<float*>(s_mm + W * M);                   // [W][M] sums of squares

  const int nt = (int)blockIdx.x - nt_first;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 4, j = lane & 15;

  // x first (a few KB, normally in L2), then the weights, so that the min/max and quantise passes
  // run while the weights are on their way from HBM.
  const int groups = K >> 3;
  // kNorm at M = 1 with ldx < 0 (a row stride has no use at M = 1): x is a table of -ldx rows of K floats, the
  // delta argument points to an int64 row number instead, and the input row is that row of the table (the number
  // clamped to it); workgroup 0 copies the row to sum_out. The decoder's first launch of a token reads the
  // token's embedding this way instead of behind a gather launch. Both arguments arrive preloaded, so a launch
  // that gathers nothing does not wait for anything new.
  const float* xin = x;
  bool gathered = false;
  if constexpr (kNorm && M == 1) {
    if (ldx < 0) {
      long id = load_global<int64_t>(pro_delta);
      id = id < 0 ? 0 : (id >= -ldx ? -ldx - 1 : id);
      xin = x + (size_t)id * K;
      pro_delta = nullptr;
      gathered = true;
    }
  }
  float xv[M][kFusedR][8];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const float* row = xin + (size_t)m * ldx;
#pragma unroll
    for (int r = 0; r < kFusedR; ++r) {
      const int c = threadIdx.x + r * nthreads;
      const int cc = c < groups ? c : groups - 1;  // a duplicate of a real element: harmless for min/max
      const float4 v0 = *reinterpret_cast<const float4*>(row + 8 * cc);
      const float4 v1 = *reinterpret_cast<const float4*>(row + 8 * cc + 4);
      const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) xv[m][r][e] = f[e];
    }
  }
  float dv[kNorm ? M : 1][kNorm ? kFusedR : 1][8];  // delta
  if (kNorm && pro_delta) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float* row = pro_delta + (size_t)m * ldx;
#pragma unroll
      for (int r = 0; r < kFusedR; ++r) {
        const int c = threadIdx.x + r * nthreads;
        const int cc = c < groups ? c : groups - 1;
        const float4 v0 = *reinterpret_cast<const float4*>(row + 8 * cc);
        const float4 v1 = *reinterpret_cast<const float4*>(row + 8 * cc + 4);
        const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) dv[m][r][e] = f[e];
      }
    }
  }
  // The norm weight is requested here, before the weights: a CU's memory pipe returns loads in issue order, and
  // behind this workgroup's weight loads it would arrive after all of them, with the normalisation waiting for it.
  float nwv[kNorm ? kFusedR : 1][8];
  if constexpr (kNorm) {
#pragma unroll
    for (int r = 0; r < kFusedR; ++r) {
      const int c = threadIdx.x + r * nthreads;
      const int cc = c < groups ? c : groups - 1;
      const float4 v0 = *reinterpret_cast<const float4*>(pro_norm_w + 8 * cc);
      const float4 v1 = *reinterpret_cast<const float4*>(pro_norm_w + 8 * cc + 4);
      const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) nwv[r][e] = f[e];
    }
  }
  // A producer that ran split over K (gemv_kparts_kernel) leaves its result as up to three partial rows:
  // they are requested here with everything else and added up, ((r0 + r1) + r2), before the row is used.
  // Grouped kernels at M = 1 only (a consumer with parts is launched through the group table).
  // The number of parts is a template argument: as a run-time value its branches around the loads and the sums cost
  // every grouped launch 0.14 us, with or without parts.
  static_assert(kInParts == 1 || (kGrouped && M == 1), "partial input rows: grouped kernels at M = 1");
  constexpr bool kParts = kInParts > 1;
  constexpr int in_parts = kInParts;
  float pv[2][kParts ? kFusedR : 1][8];
  if constexpr (kParts) {
    const float* base = kNorm ? pro_delta : x;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      if (p + 1 >= in_parts) break;  // wavefront-uniform: a part that does not exist is not requested
      const float* row = base + (size_t)(p + 1) * K;
#pragma unroll
      for (int r = 0; r < kFusedR; ++r) {
        const int c = threadIdx.x + r * nthreads;
        const int cc = c < groups ? c : groups - 1;
        const float4 v0 = *reinterpret_cast<const float4*>(row + 8 * cc);
        const float4 v1 = *reinterpret_cast<const float4*>(row + 8 * cc + 4);
        const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) pv[p][r][e] = f[e];
      }
    }
  }
  u32x4 wq[kSets][kCPW];
  u32x2 sc[kSets][kCPW];
#pragma unroll
  for (int st = 0; st < kSets; ++st) {
    const uint8_t* tiles = (st == 0 ? packed : packed1) + (size_t)nt * KC * kTileBytes;
#pragma unroll
    for (int i = 0; i < kCPW; ++i) {
      const int kc = wave + i * W < KC ? wave + i * W : KC - 1;  // masked where used
      wq[st][i] = load_global<u32x4>(tiles + (size_t)kc * kTileBytes + 16 * lane);
      sc[st][i] = load_global<u32x2>(tiles + (size_t)kc * kTileBytes + kTileQBytes + 8 * j);
    }
  }
  // Output o = m * 16 + jj belongs to thread o when the workgroup has that many threads; its
  // rsum / bias are requested now so the epilogue does not wait on memory.
  constexpr int kOutputs = M * 16;
  float rs[kSets], bs[kSets];
#pragma unroll
  for (int st = 0; st < kSets; ++st) {
    rs[st] = 0.0f;
    bs[st] = 0.0f;
    const int n = kTileRows * nt + j;
    if (threadIdx.x < kOutputs && n < N) {
      const float* rsp = st == 0 ? rsum : reinterpret_cast<const float*>(packed1 + (size_t)NT * KC * kTileBytes);
      rs[st] = load_global<float>(rsp + n);
      bs[st] = load_global<float>(rsp + NT * kTileRows + n);
    }
  }

  if constexpr (kParts) {
#pragma unroll
    for (int r = 0; r < kFusedR; ++r) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // the sum of the parts is a Linear's output: clamped to the finite f32 range like every other one
        if constexpr (kNorm) {
          dv[0][r][e] += pv[0][r][e];
          if (in_parts > 2) dv[0][r][e] += pv[1][r][e];
          dv[0][r][e] = fminf(fmaxf(dv[0][r][e], -3.402823466e+38f), 3.402823466e+38f);
        } else {
          xv[0][r][e] += pv[0][r][e];
          if (in_parts > 2) xv[0][r][e] += pv[1][r][e];
          xv[0][r][e] = fminf(fmaxf(xv[0][r][e], -3.402823466e+38f), 3.402823466e+38f);
        }
      }
    }
  }
  if (kNorm) {
    // complete the row, sum its squares, normalise: all before the quantiser sees it
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float ss = 0.0f;
#pragma unroll
      for (int r = 0; r < kFusedR; ++r) {
        const int c = threadIdx.x + r * nthreads;
        if (pro_delta) {
#pragma unroll
          for (int e = 0; e < 8; ++e) xv[m][r][e] += dv[m][r][e];
          if (pro_sum_out && blockIdx.x == 0 && c < groups) {
            float* dst = pro_sum_out + (size_t)m * ldx + 8 * c;
            *reinterpret_cast<float4*>(dst) = make_float4(xv[m][r][0], xv[m][r][1], xv[m][r][2], xv[m][r][3]);
            *reinterpret_cast<float4*>(dst + 4) = make_float4(xv[m][r][4], xv[m][r][5], xv[m][r][6], xv[m][r][7]);
          }
        } else if (gathered && pro_sum_out && blockIdx.x == 0 && c < groups) {
          float* dst = pro_sum_out + 8 * c;  // the row itself: the residual stream starts with it
          *reinterpret_cast<float4*>(dst) = make_float4(xv[m][r][0], xv[m][r][1], xv[m][r][2], xv[m][r][3]);
          *reinterpret_cast<float4*>(dst + 4) = make_float4(xv[m][r][4], xv[m][r][5], xv[m][r][6], xv[m][r][7]);
        }
        if (c < groups) {
#pragma unroll
          for (int e = 0; e < 8; ++e) ss += xv[m][r][e] * xv[m][r][e];
        }
      }
      ss = wave_sum_to_lane63(ss);
      if (lane == 63) s_ss[wave * M + m] = ss;
    }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float part = j < W ? s_ss[j * M + m] : 0.0f;
      const float total = row16_sum_all(part);
      const float rstd = 1.0f / sqrtf(total / (float)K + pro_eps);
#pragma unroll
      for (int r = 0; r < kFusedR; ++r) {
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[m][r][e] = xv[m][r][e] * (nwv[r][e] * rstd);
      }
    }
  }

#pragma unroll
  for (int m = 0; m < M; ++m) {
    float lo = xv[m][0][0], hi = xv[m][0][0];
#pragma unroll
    for (int r = 0; r < kFusedR; ++r) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        lo = fminf(lo, xv[m][r][e]);
        hi = fmaxf(hi, xv[m][r][e]);
      }
    }
    wave_minmax_pair(lo, hi);
    if (lane == 63) s_mm[wave * M + m] = make_float2(lo, hi);
  }
  __syncthreads();

  RowQuant par[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    // lane j of every 16-lane row fetches wavefront j's result (the last one again past W)
    float2 v = s_mm[(j < W ? j : W - 1) * M + m];
    row16_minmax_pair(v.x, v.y);
    par[m] = row_quant_params(v.x, v.y);
  }

  // Quantise into the LDS copy; the tile padding (k >= K) is 0.
  const int grp_per_row = Kp >> 3;
#pragma unroll
  for (int m = 0; m < M; ++m) {
#pragma unroll
    for (int r = 0; r < kFusedR; ++r) {
      const int c = threadIdx.x + r * nthreads;
      if (c < grp_per_row) {
        uint2 out = quant_group8(xv[m][r], par[m]);
        if (c >= groups) out = make_uint2(0, 0);
        *reinterpret_cast<uint2*>(s_a + (size_t)m * Kp + 8 * c) = out;
      }
    }
  }
  __syncthreads();

  float acc[kSets][decode_acc(M)];
#pragma unroll
  for (int st = 0; st < kSets; ++st)
#pragma unroll
    for (int m = 0; m < decode_acc(M); ++m) acc[st][m] = 0.0f;
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const bool valid = wave + i * W < KC;
    const int kc = valid ? wave + i * W : KC - 1;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int8_t* a_base = s_a + kTileK * kc + kBlockLen * d + 8 * g;
#pragma unroll
      for (int st = 0; st < kSets; ++st) {
        const uint32_t sw = sc[st][i][d >> 1];
        const uint32_t sbits = valid ? ((d & 1) ? (sw & 0xFFFF0000u) : (sw << 16)) : 0u;
        block_products<M>(wq[st][i][d], __uint_as_float(sbits), a_base, Kp, j, acc[st]);
      }
    }
  }
  // The sums of the four k-groups of a row, then across wavefronts via LDS.
#pragma unroll
  for (int st = 0; st < kSets; ++st) store_row_sums<M>(acc[st], s_red + (wave * kSets + st) * M * 16, lane);
  __syncthreads();

  //   y = (sum/16 + off * rsum[n]) * lhs_scale + bias[n], clamped to the finite f32 range
  const bool prefetched = nthreads >= kOutputs;
  for (int o = threadIdx.x; o < kOutputs; o += nthreads) {
    const int m = o >> 4;
    const int n = kTileRows * nt + (o & 15);
    if (n < N) {
      float rcp = 0.0f;
      int off = 0;
#pragma unroll
      for (int mm = 0; mm < M; ++mm) {  // compile-time indices keep the array in registers
        if (mm == m) {
          rcp = par[mm].recip;
          off = -par[mm].zp;
        }
      }
      float res[kSets];
#pragma unroll
      for (int st = 0; st < kSets; ++st) {
        float s = 0.0f;
#pragma unroll 4
        for (int w = 0; w < W; ++w) s += s_red[(w * kSets + st) * kOutputs + o];
        const float* rsp = st == 0 ? rsum : reinterpret_cast<const float*>(packed1 + (size_t)NT * KC * kTileBytes);
        const float rsn = prefetched ? rs[st] : load_global<float>(rsp + n);
        const float bsn = prefetched ? bs[st] : load_global<float>(rsp + NT * kTileRows + n);
        float v = __fmaf_rn((float)off, rsn, s * 0.0625f);
        v = __fmaf_rn(v, rcp, bsn);
        res[st] = fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
      }
      float v = res[0];
      if (kPair) {
        if (ga.pair_both) {
          *(W4_GLOBAL float*)(ga.y[1] + (size_t)m * N + n) = res[kSets - 1];
        } else {
          v = silu_mul(res[0], res[kSets - 1]);
        }
      }
      *(W4_GLOBAL float*)(y + (size_t)m * N + n) = v;
    }
  }
}

// Several decode rows (M >= kBatchedMinM) through 1..kMaxGroup Linears that share them: the whole op in one
// launch, like gemv_fused_kernel, with the rows' quantisation shared by more weights. With one tile row per
// workgroup every workgroup loads and quantises all M rows for 14 KB of weights (K = 1536): at M = 8 the row
// reads of a gate,up launch (560 workgroups x 48 KB from L2) exceed its weight bytes, and a thread quantises 48
// values before its first product. Here a workgroup is kWaves wavefronts: all of them load and quantise the
// rows ((row, 64 groups of 8) segments dealt to wavefronts), then every Wt of them take one tile row exactly as
// a workgroup of gemv_fused_kernel does (wavefront wl of a tile row holds chunks wl, wl + Wt, ...; same f32
// expression per output in the same order, so the results are bit-identical). Tile rows are numbered through
// the Linears of the group (ga.first). Eight wavefronts (two tile rows at K = 1536) measured best: gate,up at
// M = 8 13.8 -> 10.3 us, q,k,v 6.5 -> 5.1; sixteen cost more than they save (11.8 / 6.0).
//
// kR = 0: the rows arrive quantised (workspace of w4a32_quant_lhs: aq [M][K], recip, negzp) and are only
// copied into LDS; this form serves a long K (down_proj), whose f32 rows are too many to quantise per workgroup.
//
// The int8 rows lie in LDS as [32-k block][row][32 bytes]: the M rows of a block behind each other, so the 64
// lanes of a product's operand read (row lane % 16, 8 bytes at 8 * (lane / 16)) cover one contiguous M * 32
// bytes. As [row][Kp], with Kp a multiple of 256 bytes, every row of a block starts in the same LDS bank
// (q,k,v at M = 8: 7.6 against 6.1 us).
constexpr int kBatchedMinM = 3;
constexpr int kBatchedStageMax = 10;  // 16-byte units of quantised rows a thread copies (kR = 0)

// min and max of kR independent pairs across the wavefront, totals in lane 63: the chains of the pairs are
// interleaved, so each DPP read finds its register at least two issue slots after its write without a wait.
#define W4_MM2(c) \
  "v_min_f32_dpp %0, %0, %0 " c "\n\tv_max_f32_dpp %1, %1, %1 " c "\n\t" \
  "v_min_f32_dpp %2, %2, %2 " c "\n\tv_max_f32_dpp %3, %3, %3 " c "\n\t"
#define W4_MM3(c) W4_MM2(c) "v_min_f32_dpp %4, %4, %4 " c "\n\tv_max_f32_dpp %5, %5, %5 " c "\n\t"
#define W4_MM_STEPS(S)                                                                         \
  "s_nop 1\n\t" S("quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf")                            \
  S("quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf") S("row_half_mirror row_mask:0xf bank_mask:0xf") \
  S("row_mirror row_mask:0xf bank_mask:0xf") S("row_bcast:15 row_mask:0xa bank_mask:0xf")      \
  S("row_bcast:31 row_mask:0xc bank_mask:0xf") "s_nop 1"
template <int kR>
__device__ __forceinline__ void wave_minmax_pairs(float (&lo)[kR], float (&hi)[kR]) {
  if constexpr (kR >= 3) {
#pragma unroll
    for (int b = 0; b + 3 <= kR; b += 3) {
      asm volatile(W4_MM_STEPS(W4_MM3)
                   : "+v"(lo[b]), "+v"(hi[b]), "+v"(lo[b + 1]), "+v"(hi[b + 1]), "+v"(lo[b + 2]), "+v"(hi[b + 2]));
    }
  }
  constexpr int kDone = kR / 3 * 3;
  if constexpr (kR - kDone == 2) {
    asm volatile(W4_MM_STEPS(W4_MM2) : "+v"(lo[kDone]), "+v"(hi[kDone]), "+v"(lo[kDone + 1]), "+v"(hi[kDone + 1]));
  } else if constexpr (kR - kDone == 1) {
    wave_minmax_pair(lo[kDone], hi[kDone]);
  }
}
#undef W4_MM_STEPS
#undef W4_MM3
#undef W4_MM2

// min and max within every 8 consecutive lanes; all 8 end up with the totals
__device__ __forceinline__ void octet_minmax_pair(float& lo, float& hi) {
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
      "s_nop 1"
      : "+v"(lo), "+v"(hi));
}

// The row quantiser of the kernels that serve several rows, on (row, segment of 64 groups of 8) tasks dealt to
// the workgroup's kWaves wavefronts: wavefront w owns tasks w, w + kWaves, ... (kR of them; xv[r] holds lane's
// group of task r, loaded by load_row_tasks). Ranges of the segments (all chains of a wavefront interleaved),
// a barrier, then the ranges and parameters of all M rows at once: lanes 8 m .. 8 m + 7 hold row m's segment
// ranges (at most 8 segments: K <= 4096), reduce them and compute the row's parameters with the standalone
// quantiser's arithmetic; a task reads its row's from lane 8 m. The int8 rows go to s_a in the
// [32-k block][row][32 bytes] layout, recip / -zp of the rows to s_par ([M] f32, [M] i32). The caller
// synchronises afterwards.
template <int M, int kR>
__device__ __forceinline__ void load_row_tasks(const float* __restrict__ x, int ldx, int K, int Kp, int kWaves,
                                               int wave, int lane, float (&xv)[kR][8]) {
  const int grp_per_row = Kp >> 3, groups = K >> 3;
  const int nseg = (grp_per_row + 63) >> 6, ntask = M * nseg;
#pragma unroll
  for (int r = 0; r < kR; ++r) {
    const int t = wave + r * kWaves;
    const int tt = t < ntask ? t : ntask - 1;     // a wavefront without a task repeats the last one (not stored)
    const int m = tt / nseg, c = (tt - m * nseg) * 64 + lane;
    const int cc = c < groups ? c : groups - 1;   // a duplicate of a real element: harmless for min / max
    const float* row = x + (size_t)m * ldx + 8 * cc;
    const float4 v0 = *reinterpret_cast<const float4*>(row);
    const float4 v1 = *reinterpret_cast<const float4*>(row + 4);
    const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) xv[r][e] = f[e];
  }
}
template <int M, int kR, int kWaves>
__device__ __forceinline__ void quantise_row_tasks(const float (&xv)[kR][8], int K, int Kp, int8_t* s_a,
                                                   float2* s_mm, float* s_par, int wave, int lane) {
  const int grp_per_row = Kp >> 3, groups = K >> 3;
  const int nseg = (grp_per_row + 63) >> 6, ntask = M * nseg;
  float lo[kR], hi[kR];
#pragma unroll
  for (int r = 0; r < kR; ++r) {
    lo[r] = xv[r][0];
    hi[r] = xv[r][0];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      lo[r] = fminf(lo[r], xv[r][e]);
      hi[r] = fmaxf(hi[r], xv[r][e]);
    }
  }
  wave_minmax_pairs<kR>(lo, hi);
#pragma unroll
  for (int r = 0; r < kR; ++r) {
    const int t = wave + r * kWaves;
    if (lane == 63 && t < ntask) s_mm[t] = make_float2(lo[r], hi[r]);
  }
  __syncthreads();
  const int pm = (lane >> 3) < M ? (lane >> 3) : M - 1, ps = (lane & 7) < nseg ? (lane & 7) : nseg - 1;
  float2 v = s_mm[pm * nseg + ps];
  octet_minmax_pair(v.x, v.y);
  const RowQuant par = row_quant_params(v.x, v.y);
  if (wave == 0 && (lane & 7) == 0 && (lane >> 3) < M) {
    s_par[lane >> 3] = par.recip;
    reinterpret_cast<int*>(s_par)[M + (lane >> 3)] = -par.zp;
  }
#pragma unroll
  for (int r = 0; r < kR; ++r) {
    const int t = wave + r * kWaves;
    if (t < ntask) {  // wavefront-uniform
      const int m = t / nseg, c = (t - m * nseg) * 64 + lane;
      RowQuant pr;
      pr.scale = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(par.scale), 8 * m));
      pr.recip = 0.0f;  // not used by the quantiser
      pr.zp = __builtin_amdgcn_readlane(par.zp, 8 * m);
      if (c < grp_per_row) {
        uint2 out = quant_group8(xv[r], pr);
        if (c >= groups) out = make_uint2(0, 0);   // the tile padding, k >= K
        *reinterpret_cast<uint2*>(s_a + ((size_t)(c >> 2) * M + m) * kBlockLen + 8 * (c & 3)) = out;
      }
    }
  }
}

template <int M, int kCPW, int kR, int kWaves>
__global__ __launch_bounds__(64 * kWaves) void gemv_batched_kernel(
    const void* __restrict__ src, int ldx, unsigned kw, const uint8_t* packed0, unsigned long long firsts,
    const uint8_t* packed1, const uint8_t* packed2, const float* __restrict__ recip,
    const int32_t* __restrict__ negzp,  // 16 dwords: preloaded
    const GroupArgs ga) {
  // As in gemv_fused_kernel, what the first loads need comes in the preloaded arguments:
  //   src    = the f32 rows (kR > 0) or the quantised rows (kR = 0, with recip and negzp)
  //   kw     = K | wavefronts per tile row << 16 | Linears << 24
  //   firsts = first[1] | first[2] << 16 | first[3] << 32 | first[4] << 48 (tile rows, see GroupArgs)
  extern __shared__ __align__(16) uint8_t smem[];
  constexpr bool kPreq = kR == 0;
  constexpr int kTasks = kPreq ? 1 : kR;
  const float* x = static_cast<const float*>(src);
  const int8_t* aq = static_cast<const int8_t*>(src);
  const int K = (int)(kw & 0xFFFFu), Wt = (int)((kw >> 16) & 31u), count = (int)(kw >> 24);
  const int KC = (K + kTileK - 1) / kTileK;
  const int first_of[kMaxGroup + 1] = {0, (int)(firsts & 0xFFFFu), (int)((firsts >> 16) & 0xFFFFu),
                                       (int)((firsts >> 32) & 0xFFFFu), (int)(firsts >> 48)};
  const int Kp = KC * kTileK;
  const int grp_per_row = Kp >> 3;
  const int nseg = (grp_per_row + 63) >> 6;       // 64-group segments per row (at most 8 when quantising here)
  const int ntask = M * nseg;
  int8_t* s_a = reinterpret_cast<int8_t*>(smem);                               // [Kp / 32][M][32]
  float* s_red = reinterpret_cast<float*>(smem + (size_t)M * Kp);               // [kWaves][M][16]
  float2* s_mm = reinterpret_cast<float2*>(s_red + kWaves * M * 16);            // [ntask] (min, max)
  float* s_par = reinterpret_cast<float*>(s_mm + (kPreq ? 0 : ntask));          // [M] recip, [M] -zp
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int g = lane >> 4, j = lane & 15;
  const int T = kWaves / Wt;                      // tile rows per workgroup
  const int tg = wave / Wt, wl = wave - tg * Wt;  // this wavefront's tile row and its place in it
  const int total = first_of[kMaxGroup];  // entries past the last Linear repeat the total

  // the rows first (a few KB, normally in L2), then the weights: loads return in issue order
  float xv[kTasks][8];
  uint4 staged[kPreq ? kBatchedStageMax : 1];
  const int units = M * (Kp >> 4);
  if constexpr (kPreq) {
#pragma unroll
    // unit u of the LDS image (16 bytes at 16 u) is row (u / 2) % M, k = 32 * ((u / 2) / M) + 16 * (u % 2): threads
    // take consecutive units, so a wavefront's LDS writes are contiguous (dealt by row, they would all fall into
    // two banks)
    for (int r = 0; r < kBatchedStageMax; ++r) {
      const int u = threadIdx.x + r * 64 * kWaves;
      staged[r] = make_uint4(0, 0, 0, 0);
      if (u < units) {
        const int m = (u >> 1) % M, k = kBlockLen * ((u >> 1) / M) + 16 * (u & 1);
        if (k < K) staged[r] = *reinterpret_cast<const uint4*>(aq + (size_t)m * K + k);
      }
    }
    if (threadIdx.x < M) {
      s_par[threadIdx.x] = recip[threadIdx.x];
      reinterpret_cast<int*>(s_par)[M + threadIdx.x] = negzp[threadIdx.x];
    }
  } else {
    load_row_tasks<M, kTasks>(x, ldx, K, Kp, kWaves, wave, lane, xv);
  }
  // which Linear this wavefront's tile row belongs to
  const int gt = (int)blockIdx.x * T + tg;
  const uint8_t* packed = packed0;
  int nt_first = 0;
  if (count > 1 && gt >= first_of[1]) {
    packed = packed1;
    nt_first = first_of[1];
  }
  if (count > 2 && gt >= first_of[2]) {
    packed = packed2;
    nt_first = first_of[2];
  }
  if (count > 3 && gt >= first_of[3]) {
    packed = ga.packed[3];
    nt_first = first_of[3];
  }
  const int nt = gt < total ? gt - nt_first : 0;   // a wavefront past the last tile row repeats one (not stored)
  const uint8_t* tiles = packed + (size_t)nt * KC * kTileBytes;
  u32x4 wq[kCPW];
  u32x2 sc[kCPW];
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const int kc = wl + i * Wt < KC ? wl + i * Wt : KC - 1;  // masked where used
    wq[i] = load_global<u32x4>(tiles + (size_t)kc * kTileBytes + 16 * lane);
    sc[i] = load_global<u32x2>(tiles + (size_t)kc * kTileBytes + kTileQBytes + 8 * j);
  }
  // Output (tile row `to` of the workgroup, row m, column jj) belongs to thread (to * M + m) * 16 + jj; its
  // rsum / bias are requested now.
  const int outputs = T * M * 16;
  float rs = 0.0f, bs = 0.0f, *oy = nullptr;
  int on = 0, oN = 0;
  bool owns = false;
  {
    const int o = threadIdx.x;
    const int to = o / (M * 16), ogt = (int)blockIdx.x * T + to;
    if (o < outputs && ogt < total) {
      const uint8_t* opk = packed0;
      int ofirst = 0, oNT = first_of[1];
      oN = ga.N[0];
      oy = ga.y[0];
      if (count > 1 && ogt >= first_of[1]) {
        opk = packed1;
        ofirst = first_of[1];
        oNT = first_of[2] - first_of[1];
        oN = ga.N[1];
        oy = ga.y[1];
      }
      if (count > 2 && ogt >= first_of[2]) {
        opk = packed2;
        ofirst = first_of[2];
        oNT = first_of[3] - first_of[2];
        oN = ga.N[2];
        oy = ga.y[2];
      }
      if (count > 3 && ogt >= first_of[3]) {
        opk = ga.packed[3];
        ofirst = first_of[3];
        oNT = first_of[4] - first_of[3];
        oN = ga.N[3];
        oy = ga.y[3];
      }
      on = kTileRows * (ogt - ofirst) + (o & 15);
      owns = true;
      // the weights' planes are requested for every output column of the padded tile row; whether the column
      // exists (on < oN, with oN from the argument segment) only matters for the store
      {
        const float* rsp = reinterpret_cast<const float*>(opk + (size_t)oNT * KC * kTileBytes);
        rs = load_global<float>(rsp + on);
        bs = load_global<float>(rsp + oNT * kTileRows + on);
      }
    }
  }

  if constexpr (kPreq) {
#pragma unroll
    for (int r = 0; r < kBatchedStageMax; ++r) {
      const int u = threadIdx.x + r * 64 * kWaves;
      if (u < units) *reinterpret_cast<uint4*>(s_a + (size_t)16 * u) = staged[r];
    }
  } else {
    quantise_row_tasks<M, kTasks, kWaves>(xv, K, Kp, s_a, s_mm, s_par, wave, lane);
  }
  __syncthreads();

  float acc[decode_acc(M)];
#pragma unroll
  for (int m = 0; m < decode_acc(M); ++m) acc[m] = 0.0f;
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const bool valid = wl + i * Wt < KC;
    const int kc = valid ? wl + i * Wt : KC - 1;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int8_t* a_base = s_a + (size_t)(4 * kc + d) * (M * kBlockLen) + 8 * g;
      const uint32_t sw = sc[i][d >> 1];
      const uint32_t sbits = valid ? ((d & 1) ? (sw & 0xFFFF0000u) : (sw << 16)) : 0u;
      block_products<M>(wq[i][d], __uint_as_float(sbits), a_base, kBlockLen, j, acc);
    }
  }
  store_row_sums<M>(acc, s_red + wave * M * 16, lane);
  __syncthreads();

  //   y = (sum/16 + off * rsum[n]) * lhs_scale + bias[n], clamped to the finite f32 range
  if (owns && on < oN) {
    const int o = threadIdx.x;
    const int to = o / (M * 16), rem = o - to * (M * 16), m = rem >> 4;
    // all reads are issued before the first add (a loop over Wt would wait for each LDS read in turn); wavefronts
    // past Wt re-read the last one and are not added
    float part[kWaves];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) part[w] = s_red[(to * Wt + (w < Wt ? w : Wt - 1)) * (M * 16) + rem];
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) sum = w < Wt ? sum + part[w] : sum;
    const float rcp = s_par[m];
    const int off = reinterpret_cast<const int*>(s_par)[M + m];
    float v = __fmaf_rn((float)off, rs, sum * 0.0625f);
    v = __fmaf_rn(v, rcp, bs);
    v = fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
    *(W4_GLOBAL float*)(oy + (size_t)m * oN + on) = v;
  }
}

// One decode row through ONE Linear with a long K, the k range dealt to kDecodeParts workgroups per tile row
// (down_proj: 96 tile rows would otherwise occupy 96 of 256 CUs with 14 wavefronts each). Workgroup
// (part p, tile row nt) quantises the row as gemv_fused_kernel does (the range needs the whole row; only
// the part's own k range is converted and kept), multiplies its chunks kc0 .. kc0 + KCp - 1 and stores
//   part 0:  (sum/16 + off * rsum[n]) * lhs_scale + bias[n]        parts 1..:  (sum/16) * lhs_scale
// to y[p][n]: the parts add up to the Linear's output (up to f32 rounding; the parts themselves are not clamped,
// the reader clamps their sum to the finite f32 range) and whoever reads it next adds them, so no workgroup
// waits for another. W wavefronts hold three chunks each (KCp <= 3 W).
// Two parts measured best for down_proj (K = 8960, N = 1536: 192 workgroups of 12 wavefronts, 4.9 us against
// 5.2 us in three parts and 6.7 us unsplit); a reader adds up to kMaxInParts partial rows.
constexpr int kDecodeParts = 2;
constexpr int kMaxInParts = 3;
template <int kFusedR>
__global__ __launch_bounds__(1024) void gemv_kparts_kernel(const float* __restrict__ x, int K, int KC, int KCp,
                                                           int W, const uint8_t* packed, int N, int NT,
                                                           float* y) {
  extern __shared__ __align__(16) uint8_t smem[];
  constexpr int kCPW = 3;
  const int p = (int)blockIdx.x / NT, nt = (int)blockIdx.x - p * NT;
  const int kc0 = p * KCp, kc1 = kc0 + KCp < KC ? kc0 + KCp : KC;
  const float* rsum = reinterpret_cast<const float*>(packed + (size_t)NT * KC * kTileBytes);
  const int nthreads = 64 * W;
  int8_t* s_a = reinterpret_cast<int8_t*>(smem);                            // [KCp * 128]
  float* s_red = reinterpret_cast<float*>(smem + (size_t)KCp * kTileK);      // [W][16]
  float2* s_mm = reinterpret_cast<float2*>(s_red + W * 16);                  // [W] (min, max)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 4, j = lane & 15;

  const int groups = K >> 3;
  float xv[kFusedR][8];
#pragma unroll
  for (int r = 0; r < kFusedR; ++r) {
    const int c = threadIdx.x + r * nthreads;
    const int cc = c < groups ? c : groups - 1;
    const float4 v0 = *reinterpret_cast<const float4*>(x + 8 * cc);
    const float4 v1 = *reinterpret_cast<const float4*>(x + 8 * cc + 4);
    const float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) xv[r][e] = f[e];
  }
  // A compute unit's vector memory pipe returns loads in the order they were issued, over all its wavefronts: every
  // wavefront puts its (small, cache-resident) row loads in before any of them queues its weight loads, or a late
  // wavefront's row would wait behind the others' weight traffic.
  __syncthreads();
  const uint8_t* tiles = packed + (size_t)nt * KC * kTileBytes;
  u32x4 wq[kCPW];
  u32x2 sc[kCPW];
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const int kc = kc0 + wave + i * W < kc1 ? kc0 + wave + i * W : kc1 - 1;  // masked where used
    wq[i] = load_global<u32x4>(tiles + (size_t)kc * kTileBytes + 16 * lane);
    sc[i] = load_global<u32x2>(tiles + (size_t)kc * kTileBytes + kTileQBytes + 8 * j);
  }
  float rs = 0.0f, bs = 0.0f;
  const int n_out = kTileRows * nt + j;
  if (p == 0 && threadIdx.x < 16 && n_out < N) {
    rs = load_global<float>(rsum + n_out);
    bs = load_global<float>(rsum + NT * kTileRows + n_out);
  }

  float lo = xv[0][0], hi = xv[0][0];
#pragma unroll
  for (int r = 0; r < kFusedR; ++r) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      lo = fminf(lo, xv[r][e]);
      hi = fmaxf(hi, xv[r][e]);
    }
  }
  wave_minmax_pair(lo, hi);
  if (lane == 63) s_mm[wave] = make_float2(lo, hi);
  __syncthreads();
  float2 v = s_mm[j < W ? j : W - 1];
  row16_minmax_pair(v.x, v.y);
  const RowQuant par = row_quant_params(v.x, v.y);

  // this part's k range into LDS (the tile padding, k >= K, is 0)
  const int c0 = kc0 * (kTileK / 8), c1 = kc1 * (kTileK / 8);
#pragma unroll
  for (int r = 0; r < kFusedR; ++r) {
    const int c = threadIdx.x + r * nthreads;
    if (c >= c0 && c < c1) {
      uint2 out = quant_group8(xv[r], par);
      if (c >= groups) out = make_uint2(0, 0);
      *reinterpret_cast<uint2*>(s_a + 8 * (c - c0)) = out;
    }
  }
  // groups of the padding that no thread owns (K not a multiple of 128: at most 15 groups of the last chunk)
  for (int c = groups + threadIdx.x; c < c1; c += nthreads) {
    if (c >= c0) *reinterpret_cast<uint2*>(s_a + 8 * (c - c0)) = make_uint2(0, 0);
  }
  __syncthreads();

  float acc[1] = {0.0f};
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const bool valid = kc0 + wave + i * W < kc1;
    const int kc = valid ? kc0 + wave + i * W : kc1 - 1;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int8_t* a_base = s_a + kTileK * (kc - kc0) + kBlockLen * d + 8 * g;
      const uint32_t sw = sc[i][d >> 1];
      const uint32_t sbits = valid ? ((d & 1) ? (sw & 0xFFFF0000u) : (sw << 16)) : 0u;
      block_products<1>(wq[i][d], __uint_as_float(sbits), a_base, 0, j, acc);
    }
  }
  store_row_sums<1>(acc, s_red + wave * 16, lane);
  __syncthreads();
  if (threadIdx.x < 16 && n_out < N) {
    float sum = 0.0f;
    for (int w = 0; w < W; ++w) sum += s_red[w * 16 + threadIdx.x];
    float out;
    if (p == 0) {
      out = __fmaf_rn((float)(-par.zp), rs, sum * 0.0625f);
      out = __fmaf_rn(out, par.recip, bs);
    } else {
      out = (sum * 0.0625f) * par.recip;
    }
    *(W4_GLOBAL float*)(y + (size_t)p * N + n_out) = out;
  }
}

// One decode row through one Linear whose input is the output of the decode attention, left by
// attention_decode_kernel<.., kDefer = true> as kS key slices per head (K = heads * 128):
//   rows [kS][K]: sum over the slice's keys of exp(score - max_s) * v      hdr [kS][heads][2]: (max_s, sum_s)
// behind each other. A thread owns 8 consecutive values of one head; it requests its piece of every slice and
// the head's headers at once and merges them as the attention kernel's last workgroup would,
//   x = (sum_s rows_s * exp(max_s - max)) / (sum_s sum_s * exp(max_s - max)),
// then the kernel goes on as gemv_fused_kernel does for a single row (range, quantise, products, epilogue).
// W wavefronts of three chunks each (KC <= 3 W), K <= 512 W.
template <int kS>
__global__ __launch_bounds__(512) void gemv_attn_rows_kernel(const float* __restrict__ part, int K, int KC, int W,
                                                             const uint8_t* packed, int N, int NT, float* y) {
  extern __shared__ __align__(16) uint8_t smem[];
  constexpr int kCPW = 3;
  const int nt = (int)blockIdx.x;
  const float* rsum = reinterpret_cast<const float*>(packed + (size_t)NT * KC * kTileBytes);
  int8_t* s_a = reinterpret_cast<int8_t*>(smem);                            // [KC * 128]
  float* s_red = reinterpret_cast<float*>(smem + (size_t)KC * kTileK);       // [W][16]
  float2* s_mm = reinterpret_cast<float2*>(s_red + W * 16);                  // [W] (min, max)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 4, j = lane & 15;

  const int groups = K >> 3, heads = K >> 7;
  const int c = threadIdx.x;
  const int cc = c < groups ? c : groups - 1;
  const float* hdr = part + (size_t)kS * K + 2 * (cc >> 4);
  float2 ml[kS];
  float4 r0[kS], r1[kS];
#pragma unroll
  for (int sl = 0; sl < kS; ++sl) ml[sl] = *reinterpret_cast<const float2*>(hdr + (size_t)sl * heads * 2);
#pragma unroll
  for (int sl = 0; sl < kS; ++sl) {
    r0[sl] = *reinterpret_cast<const float4*>(part + (size_t)sl * K + 8 * cc);
    r1[sl] = *reinterpret_cast<const float4*>(part + (size_t)sl * K + 8 * cc + 4);
  }
  // every wavefront's row loads are queued before any weight load (the memory pipe returns in order)
  __syncthreads();
  const uint8_t* tiles = packed + (size_t)nt * KC * kTileBytes;
  u32x4 wq[kCPW];
  u32x2 sc[kCPW];
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const int kc = wave + i * W < KC ? wave + i * W : KC - 1;  // masked where used
    wq[i] = load_global<u32x4>(tiles + (size_t)kc * kTileBytes + 16 * lane);
    sc[i] = load_global<u32x2>(tiles + (size_t)kc * kTileBytes + kTileQBytes + 8 * j);
  }
  float rs = 0.0f, bs = 0.0f;
  const int n_out = kTileRows * nt + j;
  if (threadIdx.x < 16 && n_out < N) {
    rs = load_global<float>(rsum + n_out);
    bs = load_global<float>(rsum + NT * kTileRows + n_out);
  }

  float xv[8];
  {
    float mm = -INFINITY;
#pragma unroll
    for (int sl = 0; sl < kS; ++sl) mm = fmaxf(mm, ml[sl].x);
    float ll = 0.0f, a[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int sl = 0; sl < kS; ++sl) {
      const float wt = ml[sl].x != -INFINITY ? __expf(ml[sl].x - mm) : 0.0f;  // a slice without keys holds zeros
      ll += ml[sl].y * wt;
      a[0] += r0[sl].x * wt; a[1] += r0[sl].y * wt; a[2] += r0[sl].z * wt; a[3] += r0[sl].w * wt;
      a[4] += r1[sl].x * wt; a[5] += r1[sl].y * wt; a[6] += r1[sl].z * wt; a[7] += r1[sl].w * wt;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) xv[e] = a[e] / ll;  // key 0 is always there: ll > 0
  }

  float lo = xv[0], hi = xv[0];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    lo = fminf(lo, xv[e]);
    hi = fmaxf(hi, xv[e]);
  }
  wave_minmax_pair(lo, hi);
  if (lane == 63) s_mm[wave] = make_float2(lo, hi);
  __syncthreads();
  float2 v = s_mm[j < W ? j : W - 1];
  row16_minmax_pair(v.x, v.y);
  const RowQuant par = row_quant_params(v.x, v.y);

  const int grp_per_row = KC * (kTileK / 8);
  if (c < grp_per_row) {
    uint2 out = quant_group8(xv, par);
    if (c >= groups) out = make_uint2(0, 0);  // the tile padding, k >= K
    *reinterpret_cast<uint2*>(s_a + 8 * c) = out;
  }
  __syncthreads();

  float acc[1] = {0.0f};
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const bool valid = wave + i * W < KC;
    const int kc = valid ? wave + i * W : KC - 1;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int8_t* a_base = s_a + kTileK * kc + kBlockLen * d + 8 * g;
      const uint32_t sw = sc[i][d >> 1];
      const uint32_t sbits = valid ? ((d & 1) ? (sw & 0xFFFF0000u) : (sw << 16)) : 0u;
      block_products<1>(wq[i][d], __uint_as_float(sbits), a_base, 0, j, acc);
    }
  }
  store_row_sums<1>(acc, s_red + wave * 16, lane);
  __syncthreads();
  if (threadIdx.x < 16 && n_out < N) {
    float sum = 0.0f;
    for (int w = 0; w < W; ++w) sum += s_red[w * 16 + threadIdx.x];
    float out = __fmaf_rn((float)(-par.zp), rs, sum * 0.0625f);
    out = __fmaf_rn(out, par.recip, bs);
    *(W4_GLOBAL float*)(y + n_out) = fminf(fmaxf(out, -3.402823466e+38f), 3.402823466e+38f);
  }
}

static int pick_waves(int KC) { return KC < 16 ? KC : 16; }

template <typename Kern>
static hipError_t raise_lds_limit(Kern kern, size_t lds, LdsLimitOnce* once) {
  if (lds <= 64 * 1024) return hipSuccess;
  return once->raise(reinterpret_cast<const void*>(kern), 160 * 1024);
}

template <int M>
static hipError_t launch_gemv_m(float* y, const uint8_t* ws, const uint8_t* packed, int K, int N,
                                hipStream_t s) {
  const WeightGeom g = weight_geom(N, K);
  const WsGeom w = ws_geom(M, K);
  const int W = pick_waves(g.KC);
  const size_t lds = (size_t)M * g.Kp + (size_t)W * M * 16 * sizeof(float) + 2 * M * sizeof(float);
  auto kern = gemv_q_kernel<M>;
  static LdsLimitOnce raised;
  if (hipError_t e = raise_lds_limit(kern, lds, &raised); e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(g.NT), dim3(64 * W), lds, s, y,
                     reinterpret_cast<const int8_t*>(ws + w.aq_off),
                     reinterpret_cast<const float*>(ws + w.scale_off),
                     reinterpret_cast<const int32_t*>(ws + w.off_off), packed, N, K, g.KC,
                     reinterpret_cast<const float*>(packed + g.rsum_off),
                     reinterpret_cast<const float*>(packed + g.bias_off));
  return hipGetLastError();
}

// Launch shape of the fused kernel: W wavefronts per workgroup, each holding CPW chunks; every
// thread owns R groups of 8 activations per row.
struct FusedPlan {
  int W, CPW, R;
};
constexpr int kMaxCPW = 5;

// Shapes that keep their chunks, activations and accumulators in registers without spilling.
constexpr bool fused_shape_ok(int M, int cpw) { return cpw <= kMaxCPW && (M == 1 || M * cpw <= 24); }

// About three chunks per wavefront: fewer wavefronts mean less dispatch time and fewer copies of
// the activation pass competing for the SIMDs, more chunks a longer serial product (measured on
// K = 1536: 4 wavefronts x 3 chunks beats 12 x 1, 6 x 2 and 3 x 4 at every grid size).
static FusedPlan fused_plan(int M, int K) {
  const int KC = (K + kTileK - 1) / kTileK;
  const int groups = KC * kTileK / 8;
  const int max_r = M == 1 ? 2 : 1;  // two groups per thread and row only fit the registers at M = 1
  const int max_w = M == 1 ? kMaxWaves : 8;  // M > 1 is compiled for 512 threads (256 VGPRs each)
  for (int cpw = 3; cpw <= kMaxCPW; ++cpw) {
    int W = (KC + cpw - 1) / cpw;
    if (W > max_w) continue;
    const int c = (KC + W - 1) / W;  // chunks per wavefront with that many ...
    W = (KC + c - 1) / c;            // ... and the fewest wavefronts that need no more
    while (W <= max_w && (groups + 64 * W - 1) / (64 * W) > max_r) ++W;
    if (W > max_w || !fused_shape_ok(M, (KC + W - 1) / W)) continue;
    return FusedPlan{W, (KC + W - 1) / W, (groups + 64 * W - 1) / (64 * W)};
  }
  return FusedPlan{0, 0, 0};
}

template <int M, int R, int CPW, bool kNorm, bool kPair>
static hipError_t launch_fused_m(const GroupArgs& ga, const float* x, int ldx, int K, int W,
                                 const RowPrologue& pro, hipStream_t s) {
  const int KC = (K + kTileK - 1) / kTileK;
  const int Kp = KC * kTileK;
  const int sets = kPair ? 2 : 1;
  const size_t lds = (size_t)M * Kp + (size_t)W * sets * M * 16 * sizeof(float) +
                     (size_t)W * M * 3 * sizeof(float);
  const dim3 grid(kPair ? ga.first[1] : ga.first[ga.count]), block(64 * W);
  // what the first loads need travels in the preloaded arguments (see the kernel)
  if (K > 0xFFFF || W > 31 || ga.in_parts > kMaxInParts || ga.first[ga.count] > 0xFFFF) return hipErrorInvalidValue;
  const unsigned kw = (unsigned)K | (unsigned)W << 16 | (unsigned)ga.count << 24;
  unsigned long long firsts = 0;
  for (int i = 1; i <= kMaxGroup; ++i) {
    firsts |= (unsigned long long)(unsigned)ga.first[i <= ga.count ? i : ga.count] << (16 * (i - 1));
  }
  auto launch = [&](auto kern, LdsLimitOnce* once) -> hipError_t {
    if (hipError_t e = raise_lds_limit(kern, lds, once); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, block, lds, s, x, ldx, kw, ga.packed[0], firsts, pro.delta, pro.norm_w,
                       ga.packed[1], ga.packed[2], pro.eps, pro.sum_out, ga);
    return hipGetLastError();
  };
  static LdsLimitOnce raised1, raisedg, raisedp2, raisedp3;
  if ((ga.count == 1 && ga.in_parts <= 1) || kPair) {
    return launch(gemv_fused_kernel<M, R, false, CPW, kNorm, kPair>, &raised1);
  }
  if constexpr (M == 1) {
    if (ga.in_parts == 2) return launch(gemv_fused_kernel<M, R, true, CPW, kNorm, false, 2>, &raisedp2);
    if (ga.in_parts == 3) return launch(gemv_fused_kernel<M, R, true, CPW, kNorm, false, 3>, &raisedp3);
  }
  if (ga.in_parts > 1) return hipErrorInvalidValue;
  return launch(gemv_fused_kernel<M, R, true, CPW, kNorm, false>, &raisedg);
}

// Launch shape of gemv_batched_kernel: `waves` wavefronts per workgroup, Wt of them per tile row (a divisor of
// waves), each holding CPW chunks; a wavefront owns R (row, segment) quantisation tasks (R = 0: the rows arrive
// quantised).
struct BatchedPlan {
  int waves, Wt, CPW, R;
};
// whole op: the kernel quantises the rows itself
static BatchedPlan batched_plan(int M, int K) {
  const BatchedPlan none{0, 0, 0, 0};
  if (M < kBatchedMinM || M > kGemvMaxM) return none;
  const int KC = (K + kTileK - 1) / kTileK;
  const int nseg = (KC * (kTileK / 8) + 63) / 64;
  if (nseg > 8) return none;                        // a row's segment ranges meet in one 8-lane reduction
  const int waves = 8;  // measured: 12 and 16 wavefronts (three / four tile rows per workgroup) are no faster
  const int R = (M * nseg + waves - 1) / waves;
  if (R > 3) return none;
  for (int Wt = 1; Wt <= waves; Wt *= 2) {
    const int cpw = (KC + Wt - 1) / Wt;
    // about three chunks per wavefront, as in gemv_fused_kernel; a thread stores at most one output, so the
    // workgroup's waves / Wt tile rows x M rows x 16 columns must not exceed its threads (a short K then runs
    // with idle wavefronts rather than more tile rows)
    if (cpw <= 3 && (waves / Wt) * M * 16 <= 64 * waves) return BatchedPlan{waves, Wt, cpw, R};
  }
  return none;
}
// rows already quantised
static BatchedPlan batched_preq_plan(int M, int K) {
  const BatchedPlan none{0, 0, 0, 0};
  if (M < kBatchedMinM || M > kGemvMaxM) return none;
  const int KC = (K + kTileK - 1) / kTileK;
  const int waves = KC > 24 ? 16 : 8, cpw_max = KC > 24 ? 5 : 3;
  if ((M * KC * (kTileK / 16) + 64 * waves - 1) / (64 * waves) > kBatchedStageMax) return none;
  if ((size_t)M * KC * kTileK > 150 * 1024) return none;
  for (int Wt = 1; Wt <= waves; Wt *= 2) {
    const int cpw = (KC + Wt - 1) / Wt;
    if (cpw <= cpw_max && (waves / Wt) * M * 16 <= 64 * waves) return BatchedPlan{waves, Wt, cpw, 0};
  }
  return none;
}

template <int M, int kWaves, int kCPW, int kR>
static hipError_t launch_batched_k(const GroupArgs& ga, const float* x, int ldx, const uint8_t* ws, int K,
                                   const BatchedPlan& p, hipStream_t s) {
  const int KC = (K + kTileK - 1) / kTileK, Kp = KC * kTileK;
  const int nseg = (Kp / 8 + 63) / 64;
  const int T = kWaves / p.Wt;
  const size_t lds = (size_t)M * Kp + (size_t)kWaves * M * 16 * sizeof(float) +
                     (kR ? (size_t)M * nseg * sizeof(float2) : 0) + (size_t)2 * M * sizeof(float);
  const dim3 grid((ga.first[ga.count] + T - 1) / T), block(64 * kWaves);
  const WsGeom w = ws_geom(M, K);
  auto kern = gemv_batched_kernel<M, kCPW, kR, kWaves>;
  static LdsLimitOnce raised;
  if (hipError_t e = raise_lds_limit(kern, lds, &raised); e != hipSuccess) return e;
  if (K > 0xFFFF || p.Wt > 31 || ga.first[ga.count] > 0xFFFF) return hipErrorInvalidValue;
  const unsigned kw = (unsigned)K | (unsigned)p.Wt << 16 | (unsigned)ga.count << 24;
  unsigned long long firsts = 0;
  for (int i = 1; i <= kMaxGroup; ++i) {
    firsts |= (unsigned long long)(unsigned)ga.first[i <= ga.count ? i : ga.count] << (16 * (i - 1));
  }
  const void* src = kR ? static_cast<const void*>(x) : static_cast<const void*>(ws + w.aq_off);
  hipLaunchKernelGGL(kern, grid, block, lds, s, src, ldx, kw, ga.packed[0], firsts, ga.packed[1], ga.packed[2],
                     ws ? reinterpret_cast<const float*>(ws + w.scale_off) : nullptr,
                     ws ? reinterpret_cast<const int32_t*>(ws + w.off_off) : nullptr, ga);
  return hipGetLastError();
}

template <int M>
static hipError_t launch_batched_m(const GroupArgs& ga, const float* x, int ldx, const uint8_t* ws, int K,
                                   const BatchedPlan& p, hipStream_t s) {
#define W4_BATCHED(w, c, r) \
  if (p.waves == w && p.CPW == c && p.R == r) return launch_batched_k<M, w, c, r>(ga, x, ldx, ws, K, p, s);
  W4_BATCHED(8, 1, 1) W4_BATCHED(8, 2, 1) W4_BATCHED(8, 3, 1)
  W4_BATCHED(8, 1, 2) W4_BATCHED(8, 2, 2) W4_BATCHED(8, 3, 2)
  W4_BATCHED(8, 1, 3) W4_BATCHED(8, 2, 3) W4_BATCHED(8, 3, 3)
  W4_BATCHED(8, 1, 0) W4_BATCHED(8, 2, 0) W4_BATCHED(8, 3, 0)
  W4_BATCHED(16, 2, 0) W4_BATCHED(16, 3, 0) W4_BATCHED(16, 4, 0) W4_BATCHED(16, 5, 0)
#undef W4_BATCHED
  return hipErrorInvalidValue;
}

static hipError_t launch_batched(const GroupArgs& ga, const float* x, int ldx, const uint8_t* ws, int M, int K,
                                 const BatchedPlan& p, hipStream_t s) {
  switch (M) {
    case 3: return launch_batched_m<3>(ga, x, ldx, ws, K, p, s);
    case 4: return launch_batched_m<4>(ga, x, ldx, ws, K, p, s);
    case 5: return launch_batched_m<5>(ga, x, ldx, ws, K, p, s);
    case 6: return launch_batched_m<6>(ga, x, ldx, ws, K, p, s);
    case 7: return launch_batched_m<7>(ga, x, ldx, ws, K, p, s);
    case 8: return launch_batched_m<8>(ga, x, ldx, ws, K, p, s);
    default: return hipErrorInvalidValue;
  }
}

// ----------------------------------------------------------------------------------------
// Wide layers: one wavefront per tile row.
// ----------------------------------------------------------------------------------------
constexpr int kWideWaves = 4;        // wavefronts per workgroup
constexpr int kWideMinTiles = 2048;  // tile rows from which this kernel is used (N >= 32768)
constexpr int kWideDepth = 4;        // chunk loads a wavefront keeps in flight

// kFused: quantise x (f32, K <= 8 * 64 * kWideWaves so one group of 8 per thread and row
// suffices) into LDS first; otherwise copy the already quantised rows from the workspace.
// kNorm (with kFused): residual add + RMSNorm of the row first, as in gemv_fused_kernel.
template <int M, bool kFused, bool kNorm>
__global__ __launch_bounds__(64 * kWideWaves) void gemv_wide_kernel(
    float* __restrict__ y, const float* __restrict__ x, int ldx, const int8_t* __restrict__ aq,
    const float* __restrict__ recip, const int32_t* __restrict__ negzp,
    const uint8_t* __restrict__ packed, int N, int K, int NT, int KC, const float* __restrict__ rsum,
    const float* __restrict__ bias, const RowPrologue pro) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int Kp = KC * kTileK;
  // From three rows on (the MFMA form of the products) the int8 rows lie as [32-k block][row][32 bytes], see
  // gemv_batched_kernel: an operand read then covers contiguous bytes instead of M rows in one bank.
  constexpr bool kInterleaved = decode_mfma(M);
  int8_t* s_a = reinterpret_cast<int8_t*>(smem);                   // [M][Kp], or [Kp / 32][M][32]
  float* s_mm = reinterpret_cast<float*>(smem + (size_t)M * Kp);   // [kWideWaves][M][2] or params

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int g = lane >> 4, j = lane & 15;
  const int wave_global = blockIdx.x * kWideWaves + wave;
  const int wave_stride = gridDim.x * kWideWaves;
  const int batches = (KC + kWideDepth - 1) / kWideDepth;  // per tile row

  // Batch (nt, b) = chunks b*kWideDepth .. +kWideDepth-1 of tile row nt; chunks past the end
  // re-read the last one and are masked out when consumed.
  auto load_batch = [&](int nt, int b, uint4 (&wq)[kWideDepth], uint2 (&sc)[kWideDepth]) {
    const uint8_t* tiles = packed + (size_t)nt * KC * kTileBytes;
#pragma unroll
    for (int i = 0; i < kWideDepth; ++i) {
      const int kc = b * kWideDepth + i < KC ? b * kWideDepth + i : KC - 1;
      wq[i] = *reinterpret_cast<const uint4*>(tiles + (size_t)kc * kTileBytes + 16 * lane);
      sc[i] = *reinterpret_cast<const uint2*>(tiles + (size_t)kc * kTileBytes + kTileQBytes + 8 * j);
    }
  };
  // The first batch is requested before the activations are touched.
  uint4 wq_cur[kWideDepth];
  uint2 sc_cur[kWideDepth];
  if (wave_global < NT) load_batch(wave_global, 0, wq_cur, sc_cur);

  float recip_m[M];
  int negzp_m[M];
  if constexpr (kFused && kInterleaved && !kNorm) {
    // the rows' quantisation on (row, segment) tasks dealt to the four wavefronts
    constexpr int kR = M;  // K <= 2048 here: at most four segments per row, 4 M tasks for four wavefronts
    float xv[kR][8];
    load_row_tasks<M, kR>(x, ldx, K, Kp, kWideWaves, wave, lane, xv);
    float2* s_seg = reinterpret_cast<float2*>(s_mm);            // [M * nseg]
    float* s_par = reinterpret_cast<float*>(s_seg + M * 4);     // [M] recip, [M] -zp
    quantise_row_tasks<M, kR, kWideWaves>(xv, K, Kp, s_a, s_seg, s_par, wave, lane);
    __syncthreads();
#pragma unroll
    for (int m = 0; m < M; ++m) {
      recip_m[m] = s_par[m];
      negzp_m[m] = reinterpret_cast<const int*>(s_par)[M + m];
    }
  } else if (kFused) {
    const int groups = K >> 3;
    float xv[M][8];
    float2* s_mm2 = reinterpret_cast<float2*>(s_mm);
    const int c = (int)threadIdx.x < groups ? threadIdx.x : groups - 1;  // duplicates: harmless for min/max
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float* src = x + (size_t)m * ldx + 8 * c;
      const float4 v0 = *reinterpret_cast<const float4*>(src);
      const float4 v1 = *reinterpret_cast<const float4*>(src + 4);
      float f[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
      if (kNorm) {
        if (pro.delta) {
          const float* dsrc = pro.delta + (size_t)m * ldx + 8 * c;
          const float4 d0 = *reinterpret_cast<const float4*>(dsrc);
          const float4 d1 = *reinterpret_cast<const float4*>(dsrc + 4);
          float dd[8] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
          // a producer that ran split over K left partial rows: ((r0 + r1) + r2), as gemv_fused_kernel adds them
          for (int p = 1; p < pro.delta_parts; ++p) {
            const float4 e0 = *reinterpret_cast<const float4*>(dsrc + (size_t)p * K);
            const float4 e1 = *reinterpret_cast<const float4*>(dsrc + (size_t)p * K + 4);
            dd[0] += e0.x; dd[1] += e0.y; dd[2] += e0.z; dd[3] += e0.w;
            dd[4] += e1.x; dd[5] += e1.y; dd[6] += e1.z; dd[7] += e1.w;
          }
          if (pro.delta_parts > 1) {  // the parts' sum is a Linear's output: clamped like every other one
#pragma unroll
            for (int e = 0; e < 8; ++e) dd[e] = fminf(fmaxf(dd[e], -3.402823466e+38f), 3.402823466e+38f);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) f[e] += dd[e];
          if (pro.sum_out && blockIdx.x == 0 && (int)threadIdx.x < groups) {
            float* dst = pro.sum_out + (size_t)m * ldx + 8 * c;
            *reinterpret_cast<float4*>(dst) = make_float4(f[0], f[1], f[2], f[3]);
            *reinterpret_cast<float4*>(dst + 4) = make_float4(f[4], f[5], f[6], f[7]);
          }
        }
        const float4 w0 = *reinterpret_cast<const float4*>(pro.norm_w + 8 * c);
        const float4 w1 = *reinterpret_cast<const float4*>(pro.norm_w + 8 * c + 4);
        const float ww[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        float ss = 0.0f;
        if ((int)threadIdx.x < groups) {
#pragma unroll
          for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
        }
        ss = wave_sum_to_lane63(ss);
        float* s_ss = s_mm + 2 * kWideWaves * M;
        if (lane == 63) s_ss[wave * M + m] = ss;
        __syncthreads();
        const float total = row16_sum_all(j < kWideWaves ? s_ss[j * M + m] : 0.0f);
        const float rstd = 1.0f / sqrtf(total / (float)K + pro.eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = f[e] * (ww[e] * rstd);
      }
      float lo = f[0], hi = f[0];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        xv[m][e] = f[e];
        lo = fminf(lo, f[e]);
        hi = fmaxf(hi, f[e]);
      }
      wave_minmax_pair(lo, hi);
      if (lane == 63) s_mm2[wave * M + m] = make_float2(lo, hi);
    }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float2 v = s_mm2[(j < kWideWaves ? j : kWideWaves - 1) * M + m];
      row16_minmax_pair(v.x, v.y);
      const RowQuant p = row_quant_params(v.x, v.y);
      recip_m[m] = p.recip;
      negzp_m[m] = -p.zp;
      if ((int)threadIdx.x < (Kp >> 3)) {
        uint2 out = quant_group8(xv[m], p);
        if ((int)threadIdx.x >= groups) out = make_uint2(0, 0);
        *reinterpret_cast<uint2*>(s_a + (size_t)m * Kp + 8 * threadIdx.x) = out;
      }
    }
  } else {
    const int vec_per_row = Kp / 16;
    for (int v = threadIdx.x; v < M * vec_per_row; v += blockDim.x) {
      // 16-byte unit v of the LDS image: row-major, or (interleaved) row (v / 2) % M at k = 32 ((v / 2) / M) + 16 (v % 2)
      const int m = kInterleaved ? (v >> 1) % M : v / vec_per_row;
      const int k = kInterleaved ? kBlockLen * ((v >> 1) / M) + 16 * (v & 1) : 16 * (v % vec_per_row);
      uint4 val = make_uint4(0, 0, 0, 0);
      if (k < K) val = *reinterpret_cast<const uint4*>(aq + (size_t)m * K + k);
      *reinterpret_cast<uint4*>(s_a + (size_t)16 * v) = val;
    }
#pragma unroll
    for (int m = 0; m < M; ++m) {
      recip_m[m] = recip[m];
      negzp_m[m] = negzp[m];
    }
  }
  __syncthreads();

  float best_v = -INFINITY;
  int best_n = 0x7fffffff;
  for (int nt = wave_global; nt < NT; nt += wave_stride) {
    const int n = kTileRows * nt + j;
    float rs = 0.0f, bs = 0.0f;
    if (lane < 16 && n < N) {
      rs = rsum[n];
      bs = bias[n];
    }
    float acc[decode_acc(M)];
#pragma unroll
    for (int m = 0; m < decode_acc(M); ++m) acc[m] = 0.0f;

    for (int b = 0; b < batches; ++b) {
      // request the next batch (of this tile row, or the first of the next one) ...
      uint4 wq_nxt[kWideDepth];
      uint2 sc_nxt[kWideDepth];
      const bool last = b + 1 == batches;
      const int nt_n = last ? nt + wave_stride : nt;
      const int b_n = last ? 0 : b + 1;
      if (nt_n < NT) {
        load_batch(nt_n, b_n, wq_nxt, sc_nxt);
      } else {
#pragma unroll
        for (int i = 0; i < kWideDepth; ++i) {
          wq_nxt[i] = make_uint4(0, 0, 0, 0);
          sc_nxt[i] = make_uint2(0, 0);
        }
      }
      // ... then multiply the current one
#pragma unroll
      for (int i = 0; i < kWideDepth; ++i) {
        const int kc = b * kWideDepth + i;
        if (kc < KC) {
          const uint32_t wv[4] = {wq_cur[i].x, wq_cur[i].y, wq_cur[i].z, wq_cur[i].w};
          const float sv[4] = {__uint_as_float(sc_cur[i].x << 16),
                               __uint_as_float(sc_cur[i].x & 0xFFFF0000u),
                               __uint_as_float(sc_cur[i].y << 16),
                               __uint_as_float(sc_cur[i].y & 0xFFFF0000u)};
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            if constexpr (kInterleaved) {
              block_products<M>(wv[d], sv[d], s_a + (size_t)(4 * kc + d) * (M * kBlockLen) + 8 * g, kBlockLen, j,
                                acc);
            } else {
              block_products<M>(wv[d], sv[d], s_a + kTileK * kc + kBlockLen * d + 8 * g, Kp, j, acc);
            }
          }
        }
      }
#pragma unroll
      for (int i = 0; i < kWideDepth; ++i) {
        wq_cur[i] = wq_nxt[i];
        sc_cur[i] = sc_nxt[i];
      }
    }
    if constexpr (decode_mfma(M)) {
      // lane (g, j) holds rows 4g..4g+3 of column j; rsum / bias of the column sit in lane j
      const float rsj = __shfl(rs, j, 64), bsj = __shfl(bs, j, 64);
      if (n < N) {
#pragma unroll
        for (int m = 0; m < M; ++m) {  // compile-time row index: negzp_m / recip_m stay in registers
          if ((m >> 2) == g) {
            float sum = acc[0];
#pragma unroll
            for (int r = 1; r < 4; ++r) sum = (m & 3) == r ? acc[r] : sum;
            float v = __fmaf_rn((float)negzp_m[m], rsj, sum * 0.0625f);
            v = __fmaf_rn(v, recip_m[m], bsj);
            v = fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
            y[(size_t)m * N + n] = v;
          }
        }
      }
    } else {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        acc[m] += __shfl_xor(acc[m], 16, 64);
        acc[m] += __shfl_xor(acc[m], 32, 64);
      }
      if (lane < 16 && n < N) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
          float v = __fmaf_rn((float)negzp_m[m], rs, acc[m] * 0.0625f);
          v = __fmaf_rn(v, recip_m[m], bs);
          v = fminf(fmaxf(v, -3.402823466e+38f), 3.402823466e+38f);
          y[(size_t)m * N + n] = v;
          if (M == 1 && (v > best_v || (v == best_v && n < best_n))) {  // columns rise: the first maximum stays
            best_v = v;
            best_n = n;
          }
        }
      }
    }
  }
  if constexpr (M == 1) {
    if (pro.amax_val) {
      // lanes 0..15 hold the candidates of their columns: the largest value, the lowest column among equals
#pragma unroll
      for (int off = 8; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best_v, off, 64);
        const int on = __shfl_xor(best_n, off, 64);
        if (ov > best_v || (ov == best_v && on < best_n)) {
          best_v = ov;
          best_n = on;
        }
      }
      if (lane == 0) {
        pro.amax_val[wave_global] = best_v;
        pro.amax_idx[wave_global] = best_n;
      }
    }
  }
}

// wavefronts (= partial results) of a wide launch for N outputs
int wide_partials(int N) {
  const int NT = (N + kTileRows - 1) / kTileRows;
  return std::min((NT + kWideWaves - 1) / kWideWaves, 1024) * kWideWaves;
}

template <int M, bool kFused, bool kNorm>
static hipError_t launch_wide(float* y, const float* x, int ldx, const uint8_t* ws,
                              const uint8_t* packed, int K, int N, const RowPrologue& pro, hipStream_t s) {
  const WeightGeom g = weight_geom(N, K);
  const WsGeom w = ws_geom(M, K);
  const size_t lds = (size_t)M * g.Kp + (size_t)kWideWaves * M * 3 * sizeof(float);
  auto kern = gemv_wide_kernel<M, kFused, kNorm>;
  static LdsLimitOnce raised;
  if (hipError_t e = raise_lds_limit(kern, lds, &raised); e != hipSuccess) return e;
  // 4 workgroups of 4 wavefronts per CU; every wavefront then walks NT / 4096 tile rows
  const int grid = std::min((g.NT + kWideWaves - 1) / kWideWaves, 1024);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kWideWaves), lds, s, y, x, ldx,
                     ws ? reinterpret_cast<const int8_t*>(ws + w.aq_off) : nullptr,
                     ws ? reinterpret_cast<const float*>(ws + w.scale_off) : nullptr,
                     ws ? reinterpret_cast<const int32_t*>(ws + w.off_off) : nullptr, packed, N, K,
                     g.NT, g.KC, reinterpret_cast<const float*>(packed + g.rsum_off),
                     reinterpret_cast<const float*>(packed + g.bias_off), pro);
  return hipGetLastError();
}

static bool wide_applies(int K, int N) {
  (void)K;
  return (N + kTileRows - 1) / kTileRows >= kWideMinTiles;
}
bool gemv_wide_applies(int K, int N) { return wide_applies(K, N); }

#define W4_DISPATCH_M(CALL)   \
  switch (M) {               \
    case 1: return CALL(1);  \
    case 2: return CALL(2);  \
    case 3: return CALL(3);  \
    case 4: return CALL(4);  \
    case 5: return CALL(5);  \
    case 6: return CALL(6);  \
    case 7: return CALL(7);  \
    case 8: return CALL(8);  \
    default: return hipErrorInvalidValue; \
  }

hipError_t launch_gemv(float* y, const uint8_t* ws, const uint8_t* packed, int M, int K, int N,
                       hipStream_t s) {
  if (wide_applies(K, N)) {
#define W4_CALL(m) (launch_wide<m, false, false>(y, nullptr, 0, ws, packed, K, N, RowPrologue{nullptr, nullptr, nullptr, 0.0f}, s))
    W4_DISPATCH_M(W4_CALL)
#undef W4_CALL
  }
  if (const BatchedPlan bp = batched_preq_plan(M, K); bp.Wt != 0) {
    GroupArgs ga{};
    ga.packed[0] = packed;
    ga.y[0] = y;
    ga.N[0] = N;
    ga.first[0] = 0;
    ga.first[1] = (N + kTileRows - 1) / kTileRows;
    ga.count = 1;
    return launch_batched(ga, nullptr, 0, ws, M, K, bp, s);
  }
#define W4_CALL(m) (launch_gemv_m<m>(y, ws, packed, K, N, s))
  W4_DISPATCH_M(W4_CALL)
#undef W4_CALL
}

bool gemv_fused_applies(int M, int K, int N) {
  // Every workgroup re-reads and re-quantises the M rows. That is cheaper than a second kernel
  // launch while the rows are small next to the workgroup's weights and each thread can hold its
  // share of them in registers.
  if (M < 1 || M > kGemvMaxM || (long)M * K > 16384) return false;
  if (wide_applies(K, N)) return K <= 8 * 64 * kWideWaves;  // one group of 8 per thread and row
  return fused_plan(M, K).W != 0;
}

template <int M, int R, bool kNorm, bool kPair>
static hipError_t launch_fused_cpw(const GroupArgs& ga, const float* x, int ldx, int K,
                                   const FusedPlan& p, const RowPrologue& pro, hipStream_t s) {
#define W4_CASE(c)                                                                  \
  case c:                                                                           \
    if constexpr (fused_shape_ok(M, c) && (!kPair || c <= 3)) {                     \
      return launch_fused_m<M, R, c, kNorm, kPair>(ga, x, ldx, K, p.W, pro, s);     \
    } else {                                                                        \
      return hipErrorInvalidValue;                                                  \
    }
  switch (p.CPW) {
    W4_CASE(1)
    W4_CASE(2)
    W4_CASE(3)
    W4_CASE(4)
    W4_CASE(5)
    default: return hipErrorInvalidValue;
  }
#undef W4_CASE
}

// norm / pair: decode extras, M = 1 only (see gemv_decode_applies)
static hipError_t launch_fused_group(const GroupArgs& ga, const float* x, int ldx, int M, int K,
                                     const RowPrologue* pro, bool pair, hipStream_t s) {
  const FusedPlan p = fused_plan(M, K);
  if (p.W == 0) return hipErrorInvalidValue;
  const RowPrologue none{nullptr, nullptr, nullptr, 0.0f};
  if (pair && !pro && M > 1) {  // two Linears of equal N on the same M rows, both outputs stored (ga.pair_both)
    if (p.R != 1 || !ga.pair_both) return hipErrorInvalidValue;
#define W4_CALL(m) (launch_fused_cpw<m, 1, false, true>(ga, x, ldx, K, p, none, s))
    W4_DISPATCH_M(W4_CALL)
#undef W4_CALL
  }
  if (pro || pair) {
    if (M != 1) return hipErrorInvalidValue;
    const RowPrologue& pr = pro ? *pro : none;
    if (p.R == 2) {
      if (pro && pair) return launch_fused_cpw<1, 2, true, true>(ga, x, ldx, K, p, pr, s);
      if (pro) return launch_fused_cpw<1, 2, true, false>(ga, x, ldx, K, p, pr, s);
      return launch_fused_cpw<1, 2, false, true>(ga, x, ldx, K, p, pr, s);
    }
    if (pro && pair) return launch_fused_cpw<1, 1, true, true>(ga, x, ldx, K, p, pr, s);
    if (pro) return launch_fused_cpw<1, 1, true, false>(ga, x, ldx, K, p, pr, s);
    return launch_fused_cpw<1, 1, false, true>(ga, x, ldx, K, p, pr, s);
  }
  if (p.R == 2) {
    if (M != 1) return hipErrorInvalidValue;
    return launch_fused_cpw<1, 2, false, false>(ga, x, ldx, K, p, none, s);
  }
#define W4_CALL(m) (launch_fused_cpw<m, 1, false, false>(ga, x, ldx, K, p, none, s))
  W4_DISPATCH_M(W4_CALL)
#undef W4_CALL
}

hipError_t launch_gemv_fused(float* y, const float* x, int ldx, const uint8_t* packed, int M, int K,
                             int N, hipStream_t s) {
  if (wide_applies(K, N)) {
#define W4_CALL(m) (launch_wide<m, true, false>(y, x, ldx, nullptr, packed, K, N, RowPrologue{nullptr, nullptr, nullptr, 0.0f}, s))
    W4_DISPATCH_M(W4_CALL)
#undef W4_CALL
  }
  GroupArgs ga{};
  ga.packed[0] = packed;
  ga.y[0] = y;
  ga.N[0] = N;
  ga.first[0] = 0;
  ga.first[1] = (N + kTileRows - 1) / kTileRows;
  ga.count = 1;
  if (const BatchedPlan bp = batched_plan(M, K); bp.Wt != 0) return launch_batched(ga, x, ldx, nullptr, M, K, bp, s);
  return launch_fused_group(ga, x, ldx, M, K, nullptr, false, s);
}

bool gemv_group_applies(int M, int K, const int* N, int count) {
  if (count < 1 || count > kMaxGroup) return false;
  for (int i = 0; i < count; ++i) {
    if (!gemv_fused_applies(M, K, N[i]) || wide_applies(K, N[i])) return false;
  }
  return true;
}

hipError_t launch_gemv_group(float* const* y, const float* x, int ldx, const uint8_t* const* packed,
                             const int* N, int count, int M, int K, hipStream_t s) {
  GroupArgs ga{};
  ga.first[0] = 0;
  for (int i = 0; i < count; ++i) {
    ga.packed[i] = packed[i];
    ga.y[i] = y[i];
    ga.N[i] = N[i];
    ga.first[i + 1] = ga.first[i] + (N[i] + kTileRows - 1) / kTileRows;
  }
  ga.count = count;
  if (const BatchedPlan bp = batched_plan(M, K); bp.Wt != 0) return launch_batched(ga, x, ldx, nullptr, M, K, bp, s);
  // one row through two Linears of equal N: the pair kernel with both outputs stored
  const FusedPlan fp = fused_plan(M, K);
  if (count == 2 && N[0] == N[1] && fp.W != 0 && fp.CPW <= 3 && fp.R == 1) {
    ga.pair_both = 1;
    return launch_fused_group(ga, x, ldx, M, K, nullptr, true, s);
  }
  return launch_fused_group(ga, x, ldx, M, K, nullptr, false, s);
}

// Parts the K-split decode kernel would leave for one row through an [N][K] Linear: kDecodeParts when K is
// long, the tile rows are few (the unsplit launch would leave most CUs idle) and the shape fits the kernel,
// else 1 (no split).
int gemv_kparts(int K, int N) {
  const int KC = (K + kTileK - 1) / kTileK, NT = (N + kTileRows - 1) / kTileRows;
  if (KC < 48 || NT > 128 || wide_applies(K, N)) return 1;
  const int KCp = (KC + kDecodeParts - 1) / kDecodeParts;
  const int W = (KCp + 2) / 3;
  if (W > kMaxWaves || (KC * (kTileK / 8) + 64 * W - 1) / (64 * W) > 3) return 1;
  return kDecodeParts;
}

hipError_t launch_gemv_kparts(float* y_parts, const float* x, const uint8_t* packed, int K, int N,
                              hipStream_t s) {
  if (gemv_kparts(K, N) != kDecodeParts) return hipErrorInvalidValue;
  const int KC = (K + kTileK - 1) / kTileK, NT = (N + kTileRows - 1) / kTileRows;
  const int KCp = (KC + kDecodeParts - 1) / kDecodeParts;
  const int W = (KCp + 2) / 3;
  const int R = (KC * (kTileK / 8) + 64 * W - 1) / (64 * W);
  const size_t lds = (size_t)KCp * kTileK + (size_t)W * 16 * sizeof(float) + (size_t)W * sizeof(float2);
  const dim3 grid(NT * kDecodeParts), block(64 * W);
#define W4_KPARTS(r) \
  hipLaunchKernelGGL(gemv_kparts_kernel<r>, grid, block, lds, s, x, K, KC, KCp, W, packed, N, NT, y_parts)
  if (R == 1) W4_KPARTS(1);
  else if (R == 2) W4_KPARTS(2);
  else W4_KPARTS(3);
#undef W4_KPARTS
  return hipGetLastError();
}

// One decode row (M = 1) through 1..4 Linears with the decoder's extras: residual add + RMSNorm in
// front (norm_w != null), silu(y0) * y1 behind (pair: two Linears of equal N, result in y[0]).
bool gemv_decode_applies(int K, const int* N, int count, bool pair) {
  if (count < 1 || count > kMaxGroup || (pair && (count != 2 || N[0] != N[1]))) return false;
  const FusedPlan p = fused_plan(1, K);
  if (p.W == 0 || (pair && p.CPW > 3)) return false;
  bool wide = false;
  for (int i = 0; i < count; ++i) {
    if (!gemv_fused_applies(1, K, N[i])) return false;
    wide = wide || wide_applies(K, N[i]);
  }
  return !wide || (count == 1 && !pair);  // a wide layer goes alone
}

bool gemv_attn_rows_applies(int K, int N, int slices) {
  if (K <= 0 || N <= 0 || K % kTileK != 0 || wide_applies(K, N)) return false;
  const int KC = K / kTileK, W = (KC + 2) / 3;
  return W <= 8 && K / 8 <= 64 * W && (slices == 8 || slices == 16);
}

hipError_t launch_gemv_attn_rows(float* y, const float* part, int slices, const uint8_t* packed, int K, int N,
                                 hipStream_t s) {
  if (!gemv_attn_rows_applies(K, N, slices)) return hipErrorInvalidValue;
  const int KC = K / kTileK, NT = (N + kTileRows - 1) / kTileRows, W = (KC + 2) / 3;
  const size_t lds = (size_t)KC * kTileK + (size_t)W * 16 * sizeof(float) + (size_t)W * sizeof(float2);
  if (slices == 8) {
    hipLaunchKernelGGL(gemv_attn_rows_kernel<8>, dim3(NT), dim3(64 * W), lds, s, part, K, KC, W, packed, N, NT, y);
  } else {
    hipLaunchKernelGGL(gemv_attn_rows_kernel<16>, dim3(NT), dim3(64 * W), lds, s, part, K, KC, W, packed, N, NT, y);
  }
  return hipGetLastError();
}

hipError_t launch_gemv_decode(float* const* y, const float* x, const uint8_t* const* packed,
                              const int* N, int count, int K, const float* delta, float* sum_out,
                              const float* norm_w, float eps, bool pair, int in_parts, hipStream_t s,
                              const int64_t* x_row, int x_rows, float* amax_val, int* amax_idx) {
  RowPrologue pro{delta, sum_out, norm_w, eps, in_parts, amax_val, amax_idx};
  if (amax_val && !(count == 1 && wide_applies(K, N[0]) && amax_idx)) return hipErrorInvalidValue;
  int ldx = K;
  if (x_row) {  // a gathered row: through the norm prologue of the tile-row kernels only, no delta, no pair
    if (!norm_w || delta || x_rows <= 0 || pair || in_parts > 1) return hipErrorInvalidValue;
    for (int i = 0; i < count; ++i) {
      if (wide_applies(K, N[i])) return hipErrorInvalidValue;
    }
    pro.delta = reinterpret_cast<const float*>(x_row);  // see gemv_fused_kernel: the row number, flagged by ldx < 0
    ldx = -x_rows;
  }
  if (in_parts > 1) {
    // partial rows are added up by the grouped kernels and, in front of a norm, by the wide kernel: no pair, a
    // delta when there is a norm
    if (in_parts > kMaxInParts || pair || (norm_w && !delta)) return hipErrorInvalidValue;
    for (int i = 0; i < count; ++i) {
      if (wide_applies(K, N[i]) && !(count == 1 && norm_w)) return hipErrorInvalidValue;
    }
  }
  if (count == 1 && wide_applies(K, N[0])) {
    if (norm_w) return launch_wide<1, true, true>(y[0], x, K, nullptr, packed[0], K, N[0], pro, s);
    return launch_wide<1, true, false>(y[0], x, K, nullptr, packed[0], K, N[0], pro, s);
  }
  GroupArgs ga{};
  ga.first[0] = 0;
  for (int i = 0; i < count; ++i) {
    ga.packed[i] = packed[i];
    ga.y[i] = y[i];
    ga.N[i] = N[i];
    ga.first[i + 1] = ga.first[i] + (N[i] + kTileRows - 1) / kTileRows;
  }
  ga.count = count;
  ga.in_parts = in_parts > 1 ? in_parts : 1;
  return launch_fused_group(ga, x, ldx, 1, K, norm_w ? &pro : nullptr, pair, s);
}

}  // namespace w4
