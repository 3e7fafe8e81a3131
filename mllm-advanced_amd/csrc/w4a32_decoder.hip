// extern "C" surface of include/w4a32_decoder.h: the decoder operators and the runner that strings
// them together with the W4A32 Linears. Host code only: argument checks, state geometry, launch order.
#include "w4a32_decoder.h"

#include <algorithm>

#include "w4a32_internal.h"

namespace {

constexpr int kAttnSplit = 16;    // key slices (workgroups) per head group in the decode attention
// ... when the slices are left to the Linear that follows: 16 measured better than 8 (0.794 ms per token against
// 0.809 with the same 4 wavefronts, which then take two key blocks in sequence, and 0.810 with 8 wavefronts)
constexpr int kAttnDeferSlices = 16;
constexpr int kAttn16MinRows = 256;  // prefill rows from which the bf16-term attention kernel is the faster one
constexpr int kArgmaxBlocks = 64;
constexpr int kArgmaxParts = 4096;  // partial results an lm_head launch can leave (one per wavefront)

inline int from_hip(hipError_t e) { return e == hipSuccess ? W4A32_OK : W4A32_ELAUNCH; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline hipStream_t S(void* stream) { return static_cast<hipStream_t>(stream); }

// Scratch of the decode attention + argmax.
struct ScratchGeom {
  size_t counters_off;  // u32 [n_heads + 1]
  size_t part_off;      // f32 [n_heads][kAttnSplit][130]
  size_t amax_val_off;  // f32 [kArgmaxParts]
  size_t amax_idx_off;  // i32 [kArgmaxParts]
  size_t total;
};

ScratchGeom scratch_geom(int n_heads) {
  ScratchGeom g;
  size_t o = 0;
  g.counters_off = o;
  o = align_up(o + sizeof(unsigned int) * (n_heads + 1), 256);
  g.part_off = o;
  o = align_up(o + sizeof(float) * (size_t)n_heads * kAttnSplit * 130, 256);
  g.amax_val_off = o;
  o = align_up(o + sizeof(float) * kArgmaxParts, 256);
  g.amax_idx_off = o;
  o = align_up(o + sizeof(int) * kArgmaxParts, 256);
  g.total = o;
  return g;
}

// Everything a decoder instance keeps on the device, in one caller-owned allocation.
struct StateGeom {
  size_t pos_off, scratch_off, pfcnt_off, sin_off, cos_off, kcache_off, vcache_off;
  size_t h_off, xn_off, q_off, k_off, v_off, attn_off, delta_off, gate_off, up_off, act_off;
  size_t logits_off, ws_off, total;
  size_t cache_layer;  // floats per layer in each cache
};

size_t pf_counters(const w4a32_decoder_config* c) {
  return (size_t)c->n_heads * ((c->max_batch_tokens + 31) / 32);
}

bool config_ok(const w4a32_decoder_config* c) {
  if (!c) return false;
  if (c->hidden <= 0 || c->n_heads <= 0 || c->n_kv_heads <= 0 || c->intermediate <= 0 ||
      c->n_layers <= 0 || c->vocab <= 0 || c->max_seq <= 0 || c->max_batch_tokens <= 0)
    return false;
  if (c->head_dim != 128 || c->n_heads % c->n_kv_heads != 0) return false;
  if (c->hidden % 32 != 0 || c->intermediate % 32 != 0 || (c->n_heads * c->head_dim) % 32 != 0)
    return false;
  return true;
}

StateGeom state_geom(const w4a32_decoder_config* c) {
  StateGeom g;
  const size_t Mb = c->max_batch_tokens;
  const size_t qd = (size_t)c->n_heads * c->head_dim, kvd = (size_t)c->n_kv_heads * c->head_dim;
  size_t o = 0;
  auto take = [&](size_t bytes) {
    const size_t at = o;
    o = align_up(o + bytes, 256);
    return at;
  };
  g.pos_off = take(sizeof(int));
  g.scratch_off = take(scratch_geom(c->n_heads).total);
  // arrival counters of the prefill attention, one per (head, block of 32 queries)
  g.pfcnt_off = take(sizeof(unsigned int) * pf_counters(c));
  g.sin_off = take(sizeof(float) * c->max_seq * (c->head_dim / 2));
  g.cos_off = take(sizeof(float) * c->max_seq * (c->head_dim / 2));
  g.cache_layer = kvd * c->max_seq;
  g.kcache_off = take(sizeof(float) * g.cache_layer * c->n_layers);
  g.vcache_off = take(sizeof(float) * g.cache_layer * c->n_layers);
  g.h_off = take(sizeof(float) * Mb * c->hidden);
  g.xn_off = take(sizeof(float) * Mb * c->hidden);
  g.q_off = take(sizeof(float) * Mb * qd);
  g.k_off = take(sizeof(float) * Mb * kvd);
  g.v_off = take(sizeof(float) * Mb * kvd);
  g.attn_off = take(sizeof(float) * Mb * qd);
  g.delta_off = take(sizeof(float) * std::max<size_t>(Mb, 3) * c->hidden);  // decode: down_proj's row in partial rows (at most 3)
  g.gate_off = take(sizeof(float) * Mb * c->intermediate);
  g.up_off = take(sizeof(float) * Mb * c->intermediate);
  g.act_off = take(sizeof(float) * Mb * c->intermediate);
  g.logits_off = take(sizeof(float) * c->vocab);
  const int kmax = std::max(std::max(c->hidden, c->intermediate), (int)qd);
  g.ws_off = take(w4a32_workspace_bytes(c->max_batch_tokens, kmax));
  g.total = o;
  return g;
}

#define W4_TRY(expr)                 \
  do {                               \
    const int rc_ = (expr);          \
    if (rc_ != W4A32_OK) return rc_; \
  } while (0)

// The model on M rows that are already embedded in the residual stream `h`. Leaves the last row's
// logits in the state and the greedy token in *d_token_out. d_pos: device position of row 0.
int run_layers(const w4a32_decoder_config* c, const w4a32_decoder_weights* w, uint8_t* st,
               const StateGeom& g, int M, int64_t* d_token_out, bool advance_by_argmax, void* stream,
               int host_pos0 = -1) {
  hipStream_t s = S(stream);
  const int H = c->hidden, I = c->intermediate, D = c->head_dim;
  const int Hq = c->n_heads, Hkv = c->n_kv_heads, qd = Hq * D, kvd = Hkv * D;
  int* d_pos = reinterpret_cast<int*>(st + g.pos_off);
  uint8_t* scratch = st + g.scratch_off;
  const ScratchGeom sg = scratch_geom(Hq);
  float* h = reinterpret_cast<float*>(st + g.h_off);
  float* xn = reinterpret_cast<float*>(st + g.xn_off);
  float* q = reinterpret_cast<float*>(st + g.q_off);
  float* k = reinterpret_cast<float*>(st + g.k_off);
  float* v = reinterpret_cast<float*>(st + g.v_off);
  float* attn = reinterpret_cast<float*>(st + g.attn_off);
  float* delta = reinterpret_cast<float*>(st + g.delta_off);
  float* gate = reinterpret_cast<float*>(st + g.gate_off);
  float* up = reinterpret_cast<float*>(st + g.up_off);
  float* act = reinterpret_cast<float*>(st + g.act_off);
  float* logits = reinterpret_cast<float*>(st + g.logits_off);
  const float* sin_t = reinterpret_cast<const float*>(st + g.sin_off);
  const float* cos_t = reinterpret_cast<const float*>(st + g.cos_off);
  void* ws = st + g.ws_off;

  // gate and up (with what lies between them) as one scratch area for the operators that run while
  // both are dead
  const size_t lend = g.up_off - g.gate_off + sizeof(float) * (size_t)c->max_batch_tokens * I;
  // Prefill sizes: the operator in front of a Linear runs inside that Linear's row quantiser.
  const bool fuse_rows = M > w4::kGemvMaxM && w4::quant_rows_fusable(std::max(H, I));
  // When down_proj runs split over K, its parts are not added up by a kernel of their own: the next layer's
  // first quantiser (residual add + RMSNorm) reads them instead of `delta`. The parts lie in the gate/up
  // area, which nothing else uses between down_proj and that quantiser.
  const int down_parts = fuse_rows ? w4::splitk_plan(M, I, H).parts : 1;
  const size_t parts_bytes = down_parts > 1 ? w4a32_splitk_scratch_bytes(M, I, H) : 0;
  const bool defer_sum = down_parts > 1 && parts_bytes <= lend;
  bool delta_in_parts = false;  // the previous layer's down_proj left parts, not delta

  for (int l = 0; l < c->n_layers; ++l) {
    const w4a32_layer_weights& lw = w->layers[l];
    float* kc = reinterpret_cast<float*>(st + g.kcache_off) + (size_t)l * g.cache_layer;
    float* vc = reinterpret_cast<float*>(st + g.vcache_off) + (size_t)l * g.cache_layer;
    // h += mlp output of the previous layer; xn = norm(h)
    {
      float* ys[3] = {q, k, v};
      const void* ps[3] = {lw.q, lw.k, lw.v};
      const int ns[3] = {qd, kvd, kvd};
      if (fuse_rows) {
        if (delta_in_parts) {
          const uint8_t* down_prev = static_cast<const uint8_t*>(w->layers[l - 1].down);
          W4_TRY(from_hip(w4::launch_quant_lhs_norm_parts(h, gate, down_parts, w4::linear_bias(down_prev, H, I),
                                                          lw.attn_norm, c->rms_eps, h, M, H,
                                                          static_cast<uint8_t*>(ws), s)));
        } else {
          W4_TRY(w4a32_quant_lhs_norm(h, l == 0 ? nullptr : delta, lw.attn_norm, c->rms_eps, h, M, H, ws,
                                      stream));
        }
        W4_TRY(w4a32_matmul_quantized_grouped(ys, ws, ps, ns, 3, M, H, stream));
      } else {
        W4_TRY(from_hip(w4::launch_rmsnorm(h, l == 0 ? nullptr : delta, lw.attn_norm, M, H, c->rms_eps,
                                           h, xn, s)));
        W4_TRY(w4a32_matmul_grouped(ys, xn, ps, ns, 3, ws, M, H, stream));
      }
    }
    // a prefill knows its position on the host; from kAttn16MinRows rows on the matrix-pipe attention kernel is
    // the faster one, and its operand split does the rotation and the cache append on the way. The gate and up
    // buffers are dead here: they hold the bf16 terms of K and V.
    const bool attn16 = M > 1 && host_pos0 >= 0 && M >= kAttn16MinRows && D == 128 &&
                        w4::attention16_scratch_bytes(host_pos0 + M, Hkv) <= lend;
    if (!attn16) {
      W4_TRY(from_hip(w4::launch_rope_kv(q, k, v, sin_t, cos_t, kc, vc, M, Hq, Hkv, D, c->max_seq, d_pos,
                                         0, s)));
    }
    if (attn16) {
      W4_TRY(from_hip(w4::launch_rope_attention16(q, k, v, sin_t, cos_t, kc, vc, attn, M, Hq, Hkv, c->max_seq,
                                                  host_pos0, reinterpret_cast<uint8_t*>(gate), s)));
    } else if (M == 1) {
      W4_TRY(from_hip(w4::launch_attention_decode(
          q, kc, vc, attn, Hq, Hkv, c->max_seq, d_pos, 0, kAttnSplit,
          reinterpret_cast<float*>(scratch + sg.part_off),
          reinterpret_cast<unsigned int*>(scratch + sg.counters_off), nullptr, nullptr, nullptr, nullptr, false,
          s)));
    } else {
      // the gate and up buffers are dead here: they hold the per-chunk results of long query blocks
      W4_TRY(from_hip(w4::launch_attention_prefill(q, kc, vc, attn, M, Hq, Hkv, c->max_seq, d_pos, 0, gate,
                                                   lend, reinterpret_cast<unsigned int*>(st + g.pfcnt_off),
                                                   s)));
    }
    W4_TRY(w4a32_matmul(delta, attn, lw.o, ws, M, qd, H, stream));
    // h += attention output; xn = norm(h)
    {
      float* ys[2] = {gate, up};
      const void* ps[2] = {lw.gate, lw.up};
      const int ns[2] = {I, I};
      if (fuse_rows) {
        // gate, up, SiLU and the multiply in one launch: only silu(gate) * up is stored
        W4_TRY(w4a32_quant_lhs_norm(h, delta, lw.ffn_norm, c->rms_eps, h, M, H, ws, stream));
        W4_TRY(w4a32_matmul_quantized_silu_pair(act, ws, lw.gate, lw.up, M, H, I, stream));
      } else {
        W4_TRY(from_hip(w4::launch_rmsnorm(h, delta, lw.ffn_norm, M, H, c->rms_eps, h, xn, s)));
        W4_TRY(w4a32_matmul_grouped(ys, xn, ps, ns, 2, ws, M, H, stream));
      }
    }
    if (M > w4::kGemvMaxM) {
      if (fuse_rows) {
        W4_TRY(w4a32_quant_lhs(act, M, I, I, ws, stream));
      } else {
        W4_TRY(from_hip(w4::launch_silu_mul(gate, up, act, (size_t)M * I, s)));
        W4_TRY(w4a32_quant_lhs(act, M, I, I, ws, stream));
      }
      // few output tiles, long K: split-K, with the partial sums in the gate and up buffers,
      // which are dead once the quantised rows of silu(gate) * up exist
      delta_in_parts = defer_sum && l + 1 < c->n_layers;
      if (delta_in_parts) {
        W4_TRY(from_hip(w4::launch_gemm_splitk(nullptr, static_cast<const uint8_t*>(ws),
                                               static_cast<const uint8_t*>(lw.down), M, I, H, gate, s)));
      } else {
        W4_TRY(w4a32_matmul_quantized_splitk(delta, ws, lw.down, M, I, H, gate, lend, stream));
      }
    } else {
      W4_TRY(from_hip(w4::launch_silu_mul(gate, up, act, (size_t)M * I, s)));
      W4_TRY(w4a32_matmul(delta, act, lw.down, ws, M, I, H, stream));
    }
  }
  // Only the last row feeds the head: h_last += delta_last; xn_last = norm(h_last)
  const size_t last = (size_t)(M - 1) * H;
  W4_TRY(from_hip(w4::launch_rmsnorm(h + last, delta + last, w->final_norm, 1, H, c->rms_eps, h + last,
                                     xn + last, s)));
  if (w->lm_head_dense) {
    W4_TRY(from_hip(w4::launch_dense_rows(xn + last, H, w->lm_head_dense, w->lm_head_dense_dtype, logits, 1,
                                          c->vocab, H, s)));
  } else {
    W4_TRY(w4a32_matmul(logits, xn + last, w->lm_head, ws, 1, H, c->vocab, stream));
  }
  W4_TRY(from_hip(w4::launch_argmax(logits, c->vocab, reinterpret_cast<float*>(scratch + sg.amax_val_off),
                                    reinterpret_cast<int*>(scratch + sg.amax_idx_off),
                                    reinterpret_cast<unsigned int*>(scratch + sg.counters_off) + Hq,
                                    d_token_out, advance_by_argmax ? d_pos : nullptr, kArgmaxBlocks, s)));
  return W4A32_OK;
}

// lm_head is given, as a W4 blob or as a dense operand of a known element type that the dense kernel takes
int head_ok(const w4a32_decoder_config* c, const w4a32_decoder_weights* w) {
  if (!w->lm_head_dense) return w->lm_head ? W4A32_OK : W4A32_EINVAL;
  if (w->lm_head_dense_dtype != W4A32_DENSE_F32 && w->lm_head_dense_dtype != W4A32_DENSE_F16) return W4A32_EINVAL;
  if ((reinterpret_cast<uintptr_t>(w->lm_head_dense) & 15) != 0) return W4A32_EINVAL;
  return w4::dense_rows_applies(1, c->hidden) ? W4A32_OK : W4A32_ESHAPE;
}

// One decode row with the operators between the Linears folded into them: 5 launches per layer
// ([add+norm+q,k,v] [rope+cache+attention] [o] [add+norm+gate,up+silu*mul] [down]) instead of 9.
// The residual stream alternates between two buffers because the launch that completes a row
// (x + delta) is read by every workgroup while one of them stores the sum.
bool decode_fusable(const w4a32_decoder_config* c, bool dense_head) {
  const int qd = c->n_heads * c->head_dim, kvd = c->n_kv_heads * c->head_dim;
  const int qkv[3] = {qd, kvd, kvd}, gu[2] = {c->intermediate, c->intermediate};
  const int o[1] = {c->hidden}, head[1] = {c->vocab};
  return w4::gemv_decode_applies(c->hidden, qkv, 3, false) && w4::gemv_decode_applies(c->hidden, gu, 2, true) &&
         w4::gemv_decode_applies(qd, o, 1, false) && w4::gemv_decode_applies(c->intermediate, o, 1, false) &&
         (dense_head ? w4::dense_rows_applies(1, c->hidden) : w4::gemv_decode_applies(c->hidden, head, 1, false));
}

int run_decode_fused(const w4a32_decoder_config* c, const w4a32_decoder_weights* w, uint8_t* st,
                     const StateGeom& g, const int64_t* d_token_in, int64_t* d_token_out, void* stream) {
  hipStream_t s = S(stream);
  const int H = c->hidden, I = c->intermediate, D = c->head_dim;
  const int Hq = c->n_heads, Hkv = c->n_kv_heads, qd = Hq * D, kvd = Hkv * D;
  int* d_pos = reinterpret_cast<int*>(st + g.pos_off);
  uint8_t* scratch = st + g.scratch_off;
  const ScratchGeom sg = scratch_geom(Hq);
  float* hcur = reinterpret_cast<float*>(st + g.h_off);    // the first launch copies the token's embedding here
  float* hnext = reinterpret_cast<float*>(st + g.xn_off);
  float* q = reinterpret_cast<float*>(st + g.q_off);
  float* k = reinterpret_cast<float*>(st + g.k_off);
  float* v = reinterpret_cast<float*>(st + g.v_off);
  float* attn = reinterpret_cast<float*>(st + g.attn_off);
  float* delta = reinterpret_cast<float*>(st + g.delta_off);
  float* act = reinterpret_cast<float*>(st + g.act_off);
  float* logits = reinterpret_cast<float*>(st + g.logits_off);
  const float* sin_t = reinterpret_cast<const float*>(st + g.sin_off);
  const float* cos_t = reinterpret_cast<const float*>(st + g.cos_off);

  auto one = [&](const float* x, const void* packed, int K, int N, float* y) {
    const uint8_t* pk[1] = {static_cast<const uint8_t*>(packed)};
    float* ys[1] = {y};
    const int ns[1] = {N};
    return from_hip(w4::launch_gemv_decode(ys, x, pk, ns, 1, K, nullptr, nullptr, nullptr, 0.0f, false, 1, s));
  };

  // down_proj (K = intermediate, few tile rows) runs with its k range dealt to two workgroups per tile row;
  // its partial rows are added up by the launch that reads them: the next layer's [add+norm+q,k,v], after the
  // last layer [add+norm+lm_head].
  const int down_parts = w4::gemv_kparts(I, H);
  int delta_parts = 1;
  // The attention's key slices are merged by o_proj while it loads its row, where its shape allows: the
  // slices' workgroups then end without waiting for each other.
  const bool attn_slices_to_o = w4::gemv_attn_rows_applies(qd, H, kAttnDeferSlices);
  for (int l = 0; l < c->n_layers; ++l) {
    const w4a32_layer_weights& lw = w->layers[l];
    float* kc = reinterpret_cast<float*>(st + g.kcache_off) + (size_t)l * g.cache_layer;
    float* vc = reinterpret_cast<float*>(st + g.vcache_off) + (size_t)l * g.cache_layer;
    {
      const uint8_t* pk[3] = {static_cast<const uint8_t*>(lw.q), static_cast<const uint8_t*>(lw.k),
                              static_cast<const uint8_t*>(lw.v)};
      float* ys[3] = {q, k, v};
      const int ns[3] = {qd, kvd, kvd};
      if (l == 0) {
        // the token's row of the embedding table is gathered by this launch (and copied to hcur, where the
        // residual stream starts), not by a launch of its own
        W4_TRY(from_hip(w4::launch_gemv_decode(ys, w->embedding, pk, ns, 3, H, nullptr, hcur, lw.attn_norm,
                                               c->rms_eps, false, 1, s, d_token_in, c->vocab)));
      } else {
        W4_TRY(from_hip(w4::launch_gemv_decode(ys, hcur, pk, ns, 3, H, delta, hnext, lw.attn_norm, c->rms_eps,
                                               false, delta_parts, s)));
        std::swap(hcur, hnext);
      }
    }
    float* attn_part = reinterpret_cast<float*>(scratch + sg.part_off);
    W4_TRY(from_hip(w4::launch_attention_decode(
        q, kc, vc, attn, Hq, Hkv, c->max_seq, d_pos, 0, kAttnDeferSlices, attn_part,
        reinterpret_cast<unsigned int*>(scratch + sg.counters_off), k, v, sin_t, cos_t, attn_slices_to_o, s)));
    if (attn_slices_to_o) {
      W4_TRY(from_hip(w4::launch_gemv_attn_rows(delta, attn_part, kAttnDeferSlices, static_cast<const uint8_t*>(lw.o),
                                                qd, H, s)));
    } else {
      W4_TRY(one(attn, lw.o, qd, H, delta));
    }
    {
      const uint8_t* pk[2] = {static_cast<const uint8_t*>(lw.gate), static_cast<const uint8_t*>(lw.up)};
      float* ys[2] = {act, nullptr};
      const int ns[2] = {I, I};
      W4_TRY(from_hip(w4::launch_gemv_decode(ys, hcur, pk, ns, 2, H, delta, hnext, lw.ffn_norm, c->rms_eps,
                                             true, 1, s)));
      std::swap(hcur, hnext);
    }
    if (down_parts > 1) {
      W4_TRY(from_hip(w4::launch_gemv_kparts(delta, act, static_cast<const uint8_t*>(lw.down), I, H, s)));
      delta_parts = down_parts;
    } else {
      W4_TRY(one(act, lw.down, I, H, delta));
      delta_parts = 1;
    }
  }
  if (w->lm_head_dense) {
    // the reference's dense lm_head: residual add + final norm + the f16 / f32 rows in one launch, which also
    // leaves one (max, first column) pair per wavefront where the pairs fit
    const int parts = w4::dense_rows_partials(c->vocab);
    float* amax_val = reinterpret_cast<float*>(scratch + sg.amax_val_off);
    int* amax_idx = reinterpret_cast<int*>(scratch + sg.amax_idx_off);
    const bool pairs = parts <= kArgmaxParts;
    W4_TRY(from_hip(w4::launch_dense_head(hcur, delta, delta_parts, w->final_norm, c->rms_eps, w->lm_head_dense,
                                          w->lm_head_dense_dtype, logits, c->vocab, H, pairs ? amax_val : nullptr,
                                          pairs ? amax_idx : nullptr, s)));
    if (pairs) return from_hip(w4::launch_argmax_parts(amax_val, amax_idx, parts, d_token_out, d_pos, s));
  } else {
    const uint8_t* pk[1] = {static_cast<const uint8_t*>(w->lm_head)};
    float* ys[1] = {logits};
    const int ns[1] = {c->vocab};
    // an lm_head-sized launch leaves the first maximum of every wavefront's outputs beside the logits: the
    // greedy choice then reads a few thousand pairs instead of the whole row
    const int parts = w4::gemv_wide_applies(H, c->vocab) ? w4::wide_partials(c->vocab) : 0;
    float* amax_val = reinterpret_cast<float*>(scratch + sg.amax_val_off);
    int* amax_idx = reinterpret_cast<int*>(scratch + sg.amax_idx_off);
    if (parts > 0 && parts <= kArgmaxParts) {
      W4_TRY(from_hip(w4::launch_gemv_decode(ys, hcur, pk, ns, 1, H, delta, nullptr, w->final_norm, c->rms_eps,
                                             false, delta_parts, s, nullptr, 0, amax_val, amax_idx)));
      return from_hip(w4::launch_argmax_parts(amax_val, amax_idx, parts, d_token_out, d_pos, s));
    }
    W4_TRY(from_hip(w4::launch_gemv_decode(ys, hcur, pk, ns, 1, H, delta, nullptr, w->final_norm, c->rms_eps,
                                           false, delta_parts, s)));
  }
  return from_hip(w4::launch_argmax(logits, c->vocab, reinterpret_cast<float*>(scratch + sg.amax_val_off),
                                    reinterpret_cast<int*>(scratch + sg.amax_idx_off),
                                    reinterpret_cast<unsigned int*>(scratch + sg.counters_off) + Hq,
                                    d_token_out, d_pos, kArgmaxBlocks, s));
}

}  // namespace

extern "C" {

int w4a32_op_embedding(const int64_t* d_ids, const float* d_table, int M, int D, int vocab,
                       float* d_out, void* stream) {
  if (!d_ids || !d_table || !d_out || M <= 0 || D <= 0 || vocab <= 0) return W4A32_EINVAL;
  if (D % 4 != 0) return W4A32_ESHAPE;
  return from_hip(w4::launch_embedding(d_ids, d_table, M, D, vocab, d_out, S(stream)));
}

int w4a32_op_rmsnorm(const float* d_h, const float* d_delta, const float* d_weight, int M, int D,
                     float eps, float* d_h_out, float* d_y, void* stream) {
  if (!d_h || !d_weight || !d_y || M <= 0 || D <= 0) return W4A32_EINVAL;
  if (d_delta && !d_h_out) return W4A32_EINVAL;
  if (D % 4 != 0) return W4A32_ESHAPE;
  return from_hip(w4::launch_rmsnorm(d_h, d_delta, d_weight, M, D, eps, d_h_out, d_y, S(stream)));
}

int w4a32_op_add(const float* d_a, const float* d_b, float* d_out, size_t n, void* stream) {
  if (!d_a || !d_b || !d_out || n == 0) return W4A32_EINVAL;
  if (n % 4 != 0) return W4A32_ESHAPE;
  return from_hip(w4::launch_add(d_a, d_b, d_out, n, S(stream)));
}

int w4a32_op_silu_mul(const float* d_gate, const float* d_up, float* d_out, size_t n, void* stream) {
  if (!d_gate || !d_up || !d_out || n == 0) return W4A32_EINVAL;
  if (n % 4 != 0) return W4A32_ESHAPE;
  return from_hip(w4::launch_silu_mul(d_gate, d_up, d_out, n, S(stream)));
}

int w4a32_matmul_quantized_splitk_parts(const void* d_ws, const void* d_packed, int M, int K, int N,
                                        void* d_scratch, size_t scratch_bytes, int* parts_out, void* stream) {
  if (!d_ws || !d_packed || !d_scratch || !parts_out) return W4A32_EINVAL;
  const size_t need = w4a32_splitk_scratch_bytes(M, K, N);
  if (need == 0) return W4A32_ESHAPE;
  if (scratch_bytes < need) return W4A32_EINVAL;
  if ((reinterpret_cast<uintptr_t>(d_ws) & 255) != 0 || (reinterpret_cast<uintptr_t>(d_packed) & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(d_scratch) & 15) != 0) {
    return W4A32_EINVAL;
  }
  *parts_out = w4::splitk_plan(M, K, N).parts;
  return from_hip(w4::launch_gemm_splitk(nullptr, static_cast<const uint8_t*>(d_ws),
                                         static_cast<const uint8_t*>(d_packed), M, K, N,
                                         static_cast<float*>(d_scratch), S(stream)));
}

int w4a32_quant_lhs_norm_parts(const float* d_h, const void* d_parts, int parts, const void* d_packed,
                               int K_linear, const float* d_weight, float eps, float* d_h_out, int M, int K,
                               void* d_ws, void* stream) {
  if (!d_h || !d_parts || !d_packed || !d_weight || !d_h_out || !d_ws || M <= 0 || K <= 0 || parts < 1) {
    return W4A32_EINVAL;
  }
  if (K % 32 != 0 || K_linear <= 0 || K_linear % 32 != 0 || M <= w4::kGemvMaxM || !w4::quant_rows_fusable(K)) {
    return W4A32_ESHAPE;
  }
  if ((reinterpret_cast<uintptr_t>(d_ws) & 255) != 0 || (reinterpret_cast<uintptr_t>(d_parts) & 15) != 0) {
    return W4A32_EINVAL;
  }
  return from_hip(w4::launch_quant_lhs_norm_parts(
      d_h, static_cast<const float*>(d_parts), parts,
      w4::linear_bias(static_cast<const uint8_t*>(d_packed), K, K_linear), d_weight, eps, d_h_out, M, K,
      static_cast<uint8_t*>(d_ws), S(stream)));
}

int w4a32_quant_lhs_norm(const float* d_h, const float* d_delta, const float* d_weight, float eps,
                         float* d_h_out, int M, int K, void* d_ws, void* stream) {
  if (!d_h || !d_weight || !d_ws || M <= 0 || K <= 0) return W4A32_EINVAL;
  if (d_delta && !d_h_out) return W4A32_EINVAL;
  if (K % 32 != 0 || M <= w4::kGemvMaxM || !w4::quant_rows_fusable(K)) return W4A32_ESHAPE;
  if ((reinterpret_cast<uintptr_t>(d_ws) & 255) != 0) return W4A32_EINVAL;
  return from_hip(w4::launch_quant_lhs_norm(d_h, d_delta, d_weight, eps, d_h_out, M, K,
                                            static_cast<uint8_t*>(d_ws), S(stream)));
}

int w4a32_quant_lhs_silu_mul(const float* d_gate, const float* d_up, int M, int K, void* d_ws,
                             void* stream) {
  if (!d_gate || !d_up || !d_ws || M <= 0 || K <= 0) return W4A32_EINVAL;
  if (K % 32 != 0 || M <= w4::kGemvMaxM || !w4::quant_rows_fusable(K)) return W4A32_ESHAPE;
  if ((reinterpret_cast<uintptr_t>(d_ws) & 255) != 0) return W4A32_EINVAL;
  return from_hip(w4::launch_quant_lhs_silu_mul(d_gate, d_up, M, K, static_cast<uint8_t*>(d_ws),
                                                S(stream)));
}

int w4a32_op_rope_table(float* d_sin, float* d_cos, int max_pos, int head_dim, float base, void* stream) {
  if (!d_sin || !d_cos || max_pos <= 0 || head_dim <= 0 || !(base > 0.0f)) return W4A32_EINVAL;
  if (head_dim % 2 != 0) return W4A32_ESHAPE;
  return from_hip(w4::launch_rope_table(d_sin, d_cos, max_pos, head_dim, base, S(stream)));
}

int w4a32_op_rope_kv(float* d_q, const float* d_k, const float* d_v, const float* d_sin,
                     const float* d_cos, float* d_kcache, float* d_vcache, int M, int n_heads,
                     int n_kv_heads, int head_dim, int max_seq, const int* d_pos0, int pos0,
                     void* stream) {
  if (!d_q || !d_k || !d_v || !d_sin || !d_cos || !d_kcache || !d_vcache) return W4A32_EINVAL;
  if (M <= 0 || n_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || max_seq <= 0) return W4A32_EINVAL;
  if (head_dim % 2 != 0) return W4A32_ESHAPE;
  if (!d_pos0 && (pos0 < 0 || pos0 + M > max_seq)) return W4A32_ESHAPE;
  return from_hip(w4::launch_rope_kv(d_q, d_k, d_v, d_sin, d_cos, d_kcache, d_vcache, M, n_heads,
                                     n_kv_heads, head_dim, max_seq, d_pos0, pos0, S(stream)));
}

int w4a32_op_im2col_conv3d(const float* d_in, float* d_out, int B, int C, int T, int H, int W, int kt,
                           int kh, int kw, int st, int sh, int sw, int ld_out, void* stream) {
  if (!d_in || !d_out || B <= 0 || C <= 0 || kt <= 0 || kh <= 0 || kw <= 0 || st <= 0 || sh <= 0 || sw <= 0)
    return W4A32_EINVAL;
  if (T < kt || H < kh || W < kw) return W4A32_ESHAPE;
  if (ld_out < C * kt * kh * kw) return W4A32_ESHAPE;
  return from_hip(w4::launch_im2col_conv3d(d_in, d_out, B, C, T, H, W, kt, kh, kw, st, sh, sw, ld_out,
                                           S(stream)));
}

size_t w4a32_op_scratch_bytes(int n_heads) { return n_heads > 0 ? scratch_geom(n_heads).total : 0; }

int w4a32_op_scratch_init(void* d_scratch, int n_heads, void* stream) {
  if (!d_scratch || n_heads <= 0) return W4A32_EINVAL;
  return from_hip(w4::launch_zero_u32(static_cast<unsigned int*>(d_scratch), n_heads + 1, S(stream)));
}

int w4a32_op_attention(const float* d_q, const float* d_kcache, const float* d_vcache, float* d_out,
                       int M, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                       const int* d_pos0, int pos0, void* d_scratch, void* stream) {
  if (!d_q || !d_kcache || !d_vcache || !d_out) return W4A32_EINVAL;
  if (M <= 0 || n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0) return W4A32_EINVAL;
  if (head_dim != 128 || n_heads % n_kv_heads != 0) return W4A32_ESHAPE;
  if (!d_pos0 && (pos0 < 0 || pos0 + M > max_seq)) return W4A32_ESHAPE;
  if (M == 1 && d_scratch) {
    const ScratchGeom sg = scratch_geom(n_heads);
    uint8_t* sc = static_cast<uint8_t*>(d_scratch);
    return from_hip(w4::launch_attention_decode(
        d_q, const_cast<float*>(d_kcache), const_cast<float*>(d_vcache), d_out, n_heads, n_kv_heads,
        max_seq, d_pos0, pos0, kAttnSplit, reinterpret_cast<float*>(sc + sg.part_off),
        reinterpret_cast<unsigned int*>(sc + sg.counters_off), nullptr, nullptr, nullptr, nullptr, false,
        S(stream)));
  }
  return from_hip(w4::launch_attention_prefill(d_q, d_kcache, d_vcache, d_out, M, n_heads, n_kv_heads,
                                               max_seq, d_pos0, pos0, nullptr, 0, nullptr, S(stream)));
}

size_t w4a32_op_attention_prefill_scratch_bytes(int M, int n_heads) {
  if (M <= 0 || n_heads <= 0) return 0;
  return w4::attention_prefill_part_bytes(M, n_heads);
}

int w4a32_op_attention_prefill(const float* d_q, const float* d_kcache, const float* d_vcache,
                               float* d_out, int M, int n_heads, int n_kv_heads, int head_dim,
                               int max_seq, const int* d_pos0, int pos0, void* d_part, size_t part_bytes,
                               void* stream) {
  if (!d_q || !d_kcache || !d_vcache || !d_out) return W4A32_EINVAL;
  if (M <= 0 || n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0) return W4A32_EINVAL;
  if (head_dim != 128 || n_heads % n_kv_heads != 0) return W4A32_ESHAPE;
  if (!d_pos0 && (pos0 < 0 || pos0 + M > max_seq)) return W4A32_ESHAPE;
  if (d_part && reinterpret_cast<uintptr_t>(d_part) % 16 != 0) return W4A32_EINVAL;
  return from_hip(w4::launch_attention_prefill(d_q, d_kcache, d_vcache, d_out, M, n_heads, n_kv_heads,
                                               max_seq, d_pos0, pos0, static_cast<float*>(d_part),
                                               part_bytes, nullptr, S(stream)));
}

size_t w4a32_op_attention_prefill_bf16x3_scratch_bytes(int n_keys, int n_kv_heads) {
  if (n_keys <= 0 || n_kv_heads <= 0) return 0;
  return w4::attention16_scratch_bytes(n_keys, n_kv_heads);
}

int w4a32_op_attention_prefill_bf16x3(const float* d_q, const float* d_kcache, const float* d_vcache,
                                      float* d_out, int M, int n_heads, int n_kv_heads, int head_dim,
                                      int max_seq, int pos0, void* d_scratch, size_t scratch_bytes,
                                      void* stream) {
  if (!d_q || !d_kcache || !d_vcache || !d_out || !d_scratch) return W4A32_EINVAL;
  if (M <= 0 || n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0) return W4A32_EINVAL;
  if (head_dim != 128 || n_heads % n_kv_heads != 0) return W4A32_ESHAPE;
  if (pos0 < 0 || pos0 + M > max_seq) return W4A32_ESHAPE;
  if (reinterpret_cast<uintptr_t>(d_scratch) % 16 != 0 || reinterpret_cast<uintptr_t>(d_q) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(d_out) % 16 != 0) {
    return W4A32_EINVAL;
  }
  if (scratch_bytes < w4::attention16_scratch_bytes(pos0 + M, n_kv_heads)) return W4A32_EINVAL;
  return from_hip(w4::launch_attention16(d_q, d_kcache, d_vcache, d_out, M, n_heads, n_kv_heads, max_seq, pos0,
                                         static_cast<uint8_t*>(d_scratch), S(stream)));
}

int w4a32_op_rope_attention_prefill_bf16x3(float* d_q, const float* d_k, const float* d_v, const float* d_sin,
                                           const float* d_cos, float* d_kcache, float* d_vcache, float* d_out,
                                           int M, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                                           int pos0, void* d_scratch, size_t scratch_bytes, void* stream) {
  if (!d_q || !d_k || !d_v || !d_sin || !d_cos || !d_kcache || !d_vcache || !d_out || !d_scratch)
    return W4A32_EINVAL;
  if (M <= 0 || n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0) return W4A32_EINVAL;
  if (head_dim != 128 || n_heads % n_kv_heads != 0) return W4A32_ESHAPE;
  if (pos0 < 0 || pos0 + M > max_seq) return W4A32_ESHAPE;
  for (const void* p : {static_cast<const void*>(d_q), static_cast<const void*>(d_k),
                        static_cast<const void*>(d_v), static_cast<const void*>(d_sin),
                        static_cast<const void*>(d_cos), static_cast<const void*>(d_kcache),
                        static_cast<const void*>(d_vcache), static_cast<const void*>(d_out),
                        static_cast<const void*>(d_scratch)}) {
    if (reinterpret_cast<uintptr_t>(p) % 16 != 0) return W4A32_EINVAL;
  }
  if (scratch_bytes < w4::attention16_scratch_bytes(pos0 + M, n_kv_heads)) return W4A32_EINVAL;
  return from_hip(w4::launch_rope_attention16(d_q, d_k, d_v, d_sin, d_cos, d_kcache, d_vcache, d_out, M, n_heads,
                                              n_kv_heads, max_seq, pos0, static_cast<uint8_t*>(d_scratch),
                                              S(stream)));
}

int w4a32_op_rope_attention_decode(const float* d_q, const float* d_k, const float* d_v,
                                   const float* d_sin, const float* d_cos, float* d_kcache,
                                   float* d_vcache, float* d_out, int n_heads, int n_kv_heads,
                                   int head_dim, int max_seq, const int* d_pos0, int pos0,
                                   void* d_scratch, void* stream) {
  if (!d_q || !d_k || !d_v || !d_sin || !d_cos || !d_kcache || !d_vcache || !d_out || !d_scratch)
    return W4A32_EINVAL;
  if (n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0) return W4A32_EINVAL;
  if (head_dim != 128 || n_heads % n_kv_heads != 0) return W4A32_ESHAPE;
  if (!d_pos0 && (pos0 < 0 || pos0 >= max_seq)) return W4A32_ESHAPE;
  const ScratchGeom sg = scratch_geom(n_heads);
  uint8_t* sc = static_cast<uint8_t*>(d_scratch);
  return from_hip(w4::launch_attention_decode(
      d_q, d_kcache, d_vcache, d_out, n_heads, n_kv_heads, max_seq, d_pos0, pos0, kAttnSplit,
      reinterpret_cast<float*>(sc + sg.part_off), reinterpret_cast<unsigned int*>(sc + sg.counters_off),
      d_k, d_v, d_sin, d_cos, false, S(stream)));
}

int w4a32_op_rope_attention_decode_linear(const float* d_q, const float* d_k, const float* d_v,
                                          const float* d_sin, const float* d_cos, float* d_kcache,
                                          float* d_vcache, const void* d_packed, int N, float* d_y,
                                          int n_heads, int n_kv_heads, int head_dim, int max_seq,
                                          const int* d_pos0, int pos0, void* d_scratch, void* stream) {
  if (!d_q || !d_k || !d_v || !d_sin || !d_cos || !d_kcache || !d_vcache || !d_packed || !d_y || !d_scratch)
    return W4A32_EINVAL;
  if (n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0 || N <= 0) return W4A32_EINVAL;
  if (head_dim != 128 || n_heads % n_kv_heads != 0) return W4A32_ESHAPE;
  if (!d_pos0 && (pos0 < 0 || pos0 >= max_seq)) return W4A32_ESHAPE;
  const int K = n_heads * head_dim;
  if (!w4::gemv_attn_rows_applies(K, N, kAttnDeferSlices)) return W4A32_ESHAPE;
  const ScratchGeom sg = scratch_geom(n_heads);
  uint8_t* sc = static_cast<uint8_t*>(d_scratch);
  float* part = reinterpret_cast<float*>(sc + sg.part_off);
  W4_TRY(from_hip(w4::launch_attention_decode(
      d_q, d_kcache, d_vcache, nullptr, n_heads, n_kv_heads, max_seq, d_pos0, pos0, kAttnDeferSlices, part,
      reinterpret_cast<unsigned int*>(sc + sg.counters_off), d_k, d_v, d_sin, d_cos, true, S(stream))));
  return from_hip(w4::launch_gemv_attn_rows(d_y, part, kAttnDeferSlices, static_cast<const uint8_t*>(d_packed), K, N,
                                            S(stream)));
}

int w4a32_op_argmax(const float* d_logits, int n, void* d_scratch, int64_t* d_token,
                    int* d_pos_to_advance, void* stream) {
  if (!d_logits || !d_scratch || !d_token || n <= 0) return W4A32_EINVAL;
  // the counter slot after the per-head ones is argmax's; geometry for 1 head keeps it at index 1
  const ScratchGeom sg = scratch_geom(1);
  uint8_t* sc = static_cast<uint8_t*>(d_scratch);
  return from_hip(w4::launch_argmax(d_logits, n, reinterpret_cast<float*>(sc + sg.amax_val_off),
                                    reinterpret_cast<int*>(sc + sg.amax_idx_off),
                                    reinterpret_cast<unsigned int*>(sc + sg.counters_off) + 1, d_token,
                                    d_pos_to_advance, kArgmaxBlocks, S(stream)));
}

int w4a32_decode_linear(const w4a32_decode_linear_args* a, void* stream) {
  if (!a || !a->d_x || a->count < 1 || a->count > 4 || a->K <= 0) return W4A32_EINVAL;
  if (a->K % 32 != 0) return W4A32_ESHAPE;
  if (a->d_sum_out && (!a->d_delta || !a->d_norm_weight || a->d_sum_out == a->d_x)) return W4A32_EINVAL;
  if (a->d_delta && !a->d_norm_weight) return W4A32_EINVAL;
  const bool pair = a->silu_pair != 0;
  const uint8_t* pk[4];
  for (int i = 0; i < a->count; ++i) {
    if (!a->d_packed[i] || a->N[i] <= 0) return W4A32_EINVAL;
    if (!a->d_y[i] && !(pair && i == 1)) return W4A32_EINVAL;
    pk[i] = static_cast<const uint8_t*>(a->d_packed[i]);
  }
  if (reinterpret_cast<uintptr_t>(a->d_x) % 16 != 0) return W4A32_EINVAL;
  if (a->in_parts < 0 || a->out_parts < 0) return W4A32_EINVAL;
  if (a->out_parts > 1) {
    // one plain Linear, its result left as partial rows
    if (a->count != 1 || pair || a->d_norm_weight || a->in_parts > 1) return W4A32_EINVAL;
    if (a->out_parts != w4::gemv_kparts(a->K, a->N[0])) return W4A32_ESHAPE;
    return from_hip(w4::launch_gemv_kparts(a->d_y[0], a->d_x, pk[0], a->K, a->N[0], S(stream)));
  }
  if (!w4::gemv_decode_applies(a->K, a->N, a->count, pair)) return W4A32_ENOTSUP;
  if (a->in_parts > 1) {
    if (a->in_parts > 3 || pair || (a->d_norm_weight && !a->d_delta)) return W4A32_EINVAL;
    for (int i = 0; i < a->count; ++i) {
      // the one-wavefront-per-tile-row kernel adds partial rows only in front of a norm, for a single Linear
      if (a->N[i] >= 32768 && !(a->count == 1 && a->d_norm_weight)) return W4A32_ENOTSUP;
    }
  }
  return from_hip(w4::launch_gemv_decode(a->d_y, a->d_x, pk, a->N, a->count, a->K, a->d_delta,
                                         a->d_sum_out, a->d_norm_weight, a->norm_eps, pair, a->in_parts,
                                         S(stream)));
}

int w4a32_decode_kparts(int K, int N) {
  if (K <= 0 || N <= 0 || K % 32 != 0) return 0;
  return w4::gemv_kparts(K, N);
}

size_t w4a32_decoder_state_bytes(const w4a32_decoder_config* cfg) {
  return config_ok(cfg) ? state_geom(cfg).total : 0;
}

size_t w4a32_decoder_state_offset(const w4a32_decoder_config* cfg, int which) {
  if (!config_ok(cfg)) return 0;
  const StateGeom g = state_geom(cfg);
  switch (which) {
    case 0: return g.pos_off;
    case 1: return g.logits_off;
    case 2: return g.h_off;
    default: return 0;
  }
}

int w4a32_decoder_init(const w4a32_decoder_config* cfg, void* d_state, void* stream) {
  if (!config_ok(cfg) || !d_state) return W4A32_EINVAL;
  if (reinterpret_cast<uintptr_t>(d_state) % 256 != 0) return W4A32_EINVAL;
  const StateGeom g = state_geom(cfg);
  uint8_t* st = static_cast<uint8_t*>(d_state);
  hipStream_t s = S(stream);
  W4_TRY(from_hip(w4::launch_set_int(reinterpret_cast<int*>(st + g.pos_off), 0, s)));
  W4_TRY(from_hip(w4::launch_zero_u32(reinterpret_cast<unsigned int*>(st + g.scratch_off),
                                      cfg->n_heads + 1, s)));
  W4_TRY(from_hip(w4::launch_zero_u32(reinterpret_cast<unsigned int*>(st + g.pfcnt_off),
                                      (int)pf_counters(cfg), s)));
  return from_hip(w4::launch_rope_table(reinterpret_cast<float*>(st + g.sin_off),
                                        reinterpret_cast<float*>(st + g.cos_off), cfg->max_seq,
                                        cfg->head_dim, cfg->rope_theta, s));
}

int w4a32_decoder_prefill(const w4a32_decoder_config* cfg, const w4a32_decoder_weights* w,
                          void* d_state, const int64_t* d_tokens, int n_tokens, int pos0,
                          int64_t* d_next_token, void* stream) {
  if (!config_ok(cfg) || !w || !w->layers || !d_state || !d_tokens || !d_next_token) return W4A32_EINVAL;
  W4_TRY(head_ok(cfg, w));
  if (n_tokens <= 0 || n_tokens > cfg->max_batch_tokens) return W4A32_ESHAPE;
  if (pos0 < 0 || pos0 + n_tokens > cfg->max_seq) return W4A32_ESHAPE;
  const StateGeom g = state_geom(cfg);
  uint8_t* st = static_cast<uint8_t*>(d_state);
  hipStream_t s = S(stream);
  int* d_pos = reinterpret_cast<int*>(st + g.pos_off);
  W4_TRY(from_hip(w4::launch_set_int(d_pos, pos0, s)));
  W4_TRY(from_hip(w4::launch_embedding(d_tokens, w->embedding, n_tokens, cfg->hidden, cfg->vocab,
                                       reinterpret_cast<float*>(st + g.h_off), s)));
  W4_TRY(run_layers(cfg, w, st, g, n_tokens, d_next_token, false, stream, pos0));
  return from_hip(w4::launch_add_to_int(d_pos, n_tokens, s));
}

int w4a32_decoder_step(const w4a32_decoder_config* cfg, const w4a32_decoder_weights* w, void* d_state,
                       const int64_t* d_token_in, int64_t* d_token_out, void* stream) {
  if (!config_ok(cfg) || !w || !w->layers || !d_state || !d_token_in || !d_token_out) return W4A32_EINVAL;
  W4_TRY(head_ok(cfg, w));
  const StateGeom g = state_geom(cfg);
  uint8_t* st = static_cast<uint8_t*>(d_state);
  if (decode_fusable(cfg, w->lm_head_dense != nullptr)) return run_decode_fused(cfg, w, st, g, d_token_in, d_token_out, stream);
  W4_TRY(from_hip(w4::launch_embedding(d_token_in, w->embedding, 1, cfg->hidden, cfg->vocab,
                                       reinterpret_cast<float*>(st + g.h_off), S(stream))));
  return run_layers(cfg, w, st, g, 1, d_token_out, true, stream);
}

}  // extern "C"
