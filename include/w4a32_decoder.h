/*
 * C ABI of the f32 operators that run between the W4A32 Linears of a Qwen2-style decoder, and of a
 * decoder runner built from them (one call = prefill of a prompt, or one greedy decode step).
 * Same conventions as w4a32_hip.h: d_* pointers are device memory, calls only enqueue on
 * `stream`, nothing allocates, synchronises or exits; the return value is a W4A32_* code.
 *
 * Positions and lengths are read from device memory, so a decode step is one fixed launch
 * sequence that a caller may capture into a HIP graph and replay per token.
 */
#ifndef W4A32_DECODER_H
#define W4A32_DECODER_H

#include "w4a32_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- operators ------------------------------------------------------------------------- */

/* d_out[m][:] = d_table[d_ids[m]][:]  (f32 rows of D, int64 ids clamped to [0, vocab)).
 * LLMEmbeddingTokenOp::forward, mllm/Backends/Arm/Ops/LLMEmbeddingTokenOp.cpp:24-50. */
int w4a32_op_embedding(const int64_t* d_ids, const float* d_table, int M, int D, int vocab,
                       float* d_out, void* stream);

/* h_out = h + delta (skipped when d_delta is NULL); y = h_out * (w * 1/sqrt(mean(h_out^2) + eps)).
 * d_h_out may alias d_h. D % 4 == 0.
 * ArmRMSNormOp::forward, mllm/Backends/Arm/Ops/RMSNormOp.cpp:36-76, with the residual add of
 * QWenDecoder::forward (mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:175-183) in front. */
int w4a32_op_rmsnorm(const float* d_h, const float* d_delta, const float* d_weight, int M, int D,
                     float eps, float* d_h_out, float* d_y, void* stream);

/* out = a + b; out = silu(gate) * up (QWenMLP::forward, modeling_ds_qwen2.hpp:47-54). n % 4 == 0.
 * silu(g) * u is evaluated as g * rcp(1 + exp2(-g * log2 e)) * u with the hardware's exponential and
 * reciprocal (about 1 ulp each, 3e-7 relative against the correctly rounded expression), the same
 * expression in every kernel of this library that applies it. */
int w4a32_op_add(const float* d_a, const float* d_b, float* d_out, size_t n, void* stream);
int w4a32_op_silu_mul(const float* d_gate, const float* d_up, float* d_out, size_t n, void* stream);

/* The two operators above with the row quantiser of the Linear that reads their result behind them
 * (w4a32_quant_lhs, include/w4a32_hip.h): the f32 rows they would write are never stored, the
 * quantised rows go to d_ws for w4a32_matmul_quantized*(). For M > 8 rows of K <= 16384 values.
 *   norm:     h_out = h + delta (skipped when d_delta is NULL; d_h_out may alias d_h), then the
 *             rows h_out * (w * 1/sqrt(mean(h_out^2) + eps)) are quantised;
 *   silu_mul: the rows silu(gate) * up are quantised.
 * The reference runs RMSNormOp / the MLP's elementwise ops and the Linear's own row quantiser as
 * separate passes (RMSNormOp.cpp:36-76, modeling_ds_qwen2.hpp:47-54, kai_linear.cpp:358-362). */
int w4a32_quant_lhs_norm(const float* d_h, const float* d_delta, const float* d_weight, float eps,
                         float* d_h_out, int M, int K, void* d_ws, void* stream);
int w4a32_quant_lhs_silu_mul(const float* d_gate, const float* d_up, int M, int K, void* d_ws,
                             void* stream);

/* A Linear that runs split over K (w4a32_splitk_scratch_bytes(M, K, N) != 0, include/w4a32_hip.h) followed by
 * the residual add and the next RMSNorm + row quantiser, without the kernel that adds the parts up:
 *   w4a32_matmul_quantized_splitk_parts leaves *parts_out partial products [parts][M][N] in d_scratch (at
 *     least w4a32_splitk_scratch_bytes bytes), each already carrying the row and column factors of the
 *     Linear's output transform; W4A32_ESHAPE when the library does not split this problem;
 *   w4a32_quant_lhs_norm_parts is w4a32_quant_lhs_norm with delta = ((part 0 + part 1) + ...) + bias of
 *     that Linear (d_packed, N_linear = this call's K, K_linear), clamped to the finite f32 range like
 *     every Linear output.
 * Same operators as above (the MLP's down_proj, the decoder layer's residual add and the next layer's
 * input_layer_norm_: modeling_ds_qwen2.hpp:47-54, :175-183); the sum differs from w4a32_matmul_quantized_splitk's
 * in f32 rounding only (the factors are applied before the parts are added instead of after). */
int w4a32_matmul_quantized_splitk_parts(const void* d_ws, const void* d_packed, int M, int K, int N,
                                        void* d_scratch, size_t scratch_bytes, int* parts_out, void* stream);
int w4a32_quant_lhs_norm_parts(const float* d_h, const void* d_parts, int parts, const void* d_packed,
                               int K_linear, const float* d_weight, float eps, float* d_h_out, int M, int K,
                               void* d_ws, void* stream);

/* sin/cos tables [max_pos][head_dim/2]: theta = pos / base^(2d/head_dim).
 * precompute_normal_hf_sin_cos, mllm/Backends/Arm/Kernels/rope.cpp:20-37. */
int w4a32_op_rope_table(float* d_sin, float* d_cos, int max_pos, int head_dim, float base,
                        void* stream);

/* Rotates q [M][n_heads*head_dim] in place, rotates k and copies v [M][n_kv_heads*head_dim] into the
 * caches [n_kv_heads][max_seq][head_dim] at positions pos0 + m. pos0 = *d_pos0 when d_pos0 is not
 * NULL, else the argument. normal_hf_rope (rope.cpp:39-80) + ArmKVCacheOp::forward
 * (mllm/Backends/Arm/Ops/KVCacheOp.cpp:44-72; the reference's head-repeated copies are not stored). */
int w4a32_op_rope_kv(float* d_q, const float* d_k, const float* d_v, const float* d_sin,
                     const float* d_cos, float* d_kcache, float* d_vcache, int M, int n_heads,
                     int n_kv_heads, int head_dim, int max_seq, const int* d_pos0, int pos0,
                     void* stream);

/* im2col of a Conv3D without padding or dilation: d_in [B][C][T][H][W] -> d_out [B*OT*OH*OW][ld_out] with
 * column (c, kt, kh, kw) at c*kt*kh*kw + ..., O* = (size - kernel) / stride + 1; columns from C*kt*kh*kw up
 * to ld_out are written as zeros (pad K to a multiple of 32 and zero-pad the weight rows alike: the
 * convolution is then w4a32_matmul on d_out, as ArmConv3DOp::forward does it,
 * mllm/Backends/Arm/Ops/Conv3DOp.cpp:48-188 with mllm/Backends/Arm/Kernels/conv3d.cpp:15-78). The result
 * rows are [b][ot][oh][ow] x out_channels, i.e. channels-last. */
int w4a32_op_im2col_conv3d(const float* d_in, float* d_out, int B, int C, int T, int H, int W, int kt,
                           int kh, int kw, int st, int sh, int sw, int ld_out, void* stream);

/* Scratch of the decode attention and of argmax: arrival counters + partial results. Must be cleared
 * once with w4a32_op_scratch_init before its first use; the kernels leave it cleared. */
size_t w4a32_op_scratch_bytes(int n_heads);
int w4a32_op_scratch_init(void* d_scratch, int n_heads, void* stream);

/* out[m][h][:] = softmax(q[m][h] . K[0..pos0+m] / sqrt(head_dim)) V, head h reading KV head
 * h / (n_heads / n_kv_heads). head_dim must be 128. With M == 1 and d_scratch given, the keys are split
 * over several wavefronts per head (decode); otherwise one wavefront per (head, query).
 * QWenAttention::forward, modeling_ds_qwen2.hpp:133-151 (matmul, CausalMaskOp.cpp:22-71,
 * SoftmaxOp.cpp:18-50, matmul). */
int w4a32_op_attention(const float* d_q, const float* d_kcache, const float* d_vcache, float* d_out,
                       int M, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                       const int* d_pos0, int pos0, void* d_scratch, void* stream);

/* The same operator for M > 1 rows with scratch lent by the caller: with at least
 * w4a32_op_attention_prefill_scratch_bytes(M, n_heads) bytes at d_part (16-byte aligned; contents need
 * not be kept or cleared) and at most 128 (head, block of 32 queries) pairs, the keys of a query block are
 * dealt to up to 8 workgroups and the last of them to finish combines their results (short prompts, or few
 * rows that continue a long context, would otherwise use a fraction of the CUs; the arrival counters at the
 * head of d_part are cleared by a small launch first); else it runs as w4a32_op_attention does. */
size_t w4a32_op_attention_prefill_scratch_bytes(int M, int n_heads);
int w4a32_op_attention_prefill(const float* d_q, const float* d_kcache, const float* d_vcache,
                               float* d_out, int M, int n_heads, int n_kv_heads, int head_dim,
                               int max_seq, const int* d_pos0, int pos0, void* d_part, size_t part_bytes,
                               void* stream);

/* The same operator for M >= 32 rows at a position the host knows, with both products on the 16-bit matrix
 * pipe at f32 accuracy: every f32 operand is split into three bf16 terms and a product is the six partial
 * products that matter (v_mfma_f32_32x32x16_bf16, f32 accumulation; 2.7 x the rate of the f32 matrix
 * instruction, same exponent range as f32, error below 2^-22 of |x||y| per product). A first launch splits K and V
 * of keys [0, pos0 + M) (V transposed) into d_scratch: at least
 * w4a32_op_attention_prefill_bf16x3_scratch_bytes(pos0 + M, n_kv_heads) bytes, 16-byte aligned, contents need
 * not be kept. Same reference operator as w4a32_op_attention (modeling_ds_qwen2.hpp:133-151). */
size_t w4a32_op_attention_prefill_bf16x3_scratch_bytes(int n_keys, int n_kv_heads);
int w4a32_op_attention_prefill_bf16x3(const float* d_q, const float* d_kcache, const float* d_vcache,
                                      float* d_out, int M, int n_heads, int n_kv_heads, int head_dim,
                                      int max_seq, int pos0, void* d_scratch, size_t scratch_bytes,
                                      void* stream);

/* w4a32_op_rope_kv (position given on the host) followed by w4a32_op_attention_prefill_bf16x3, in two launches
 * instead of three: the launch that splits K and V into bf16 terms also rotates q (in place) and the new rows of
 * k, and appends k and v to the caches. d_q, d_k, d_v are the un-rotated outputs of the q/k/v Linears for rows
 * at positions pos0 .. pos0 + M - 1. Caches, d_q and d_out end up bit-identical to the two operators in
 * sequence. normal_hf_rope (rope.cpp:39-80), ArmKVCacheOp::forward (KVCacheOp.cpp:44-72) and the attention of
 * modeling_ds_qwen2.hpp:133-151. Scratch as for w4a32_op_attention_prefill_bf16x3. */
int w4a32_op_rope_attention_prefill_bf16x3(float* d_q, const float* d_k, const float* d_v, const float* d_sin,
                                           const float* d_cos, float* d_kcache, float* d_vcache, float* d_out,
                                           int M, int n_heads, int n_kv_heads, int head_dim, int max_seq,
                                           int pos0, void* d_scratch, size_t scratch_bytes, void* stream);

/* Decode step (one token at position pos0) with w4a32_op_rope_kv folded into the attention launch:
 * d_q, d_k, d_v are the un-rotated outputs of the q/k/v Linears; the kernel rotates q and k, appends k
 * and v to the caches at pos0 and attends over keys 0..pos0. Same results as the two operators in
 * sequence (d_q itself is left un-rotated). */
int w4a32_op_rope_attention_decode(const float* d_q, const float* d_k, const float* d_v,
                                   const float* d_sin, const float* d_cos, float* d_kcache,
                                   float* d_vcache, float* d_out, int n_heads, int n_kv_heads,
                                   int head_dim, int max_seq, const int* d_pos0, int pos0,
                                   void* d_scratch, void* stream);

/* The same decode step followed by the Linear that reads the attention output (o_proj: K = n_heads *
 * head_dim inputs, N outputs, d_packed from w4a32_quant_pack_rhs), as the decoder's step issues the two:
 * the attention launch leaves its key slices unmerged and the Linear merges them while it loads its input
 * row, so no workgroup of the attention waits for another. d_y [N] receives what
 * w4a32_op_rope_attention_decode followed by w4a32_matmul (M = 1) would, bit for bit; the attention output
 * itself is not materialised. W4A32_ESHAPE when the Linear's shape has no such kernel (K > 3072, or an
 * lm_head-sized N): then call the two operators.
 * Reference: the attention block of modeling_ds_qwen2.hpp:126-153 followed by o_proj (:154). */
int w4a32_op_rope_attention_decode_linear(const float* d_q, const float* d_k, const float* d_v,
                                          const float* d_sin, const float* d_cos, float* d_kcache,
                                          float* d_vcache, const void* d_packed, int N, float* d_y,
                                          int n_heads, int n_kv_heads, int head_dim, int max_seq,
                                          const int* d_pos0, int pos0, void* d_scratch, void* stream);

/* *d_token = index of the first maximum of d_logits[0..n) (AutoLLM.hpp:70-88); when d_pos_to_advance
 * is not NULL, *d_pos_to_advance += 1 afterwards. */
int w4a32_op_argmax(const float* d_logits, int n, void* d_scratch, int64_t* d_token,
                    int* d_pos_to_advance, void* stream);

/* One decode row (M = 1) through 1..4 W4A32 Linears that share it, with the operators around them
 * folded into the same launch:
 *   in front  (d_norm_weight != NULL): row = d_x + d_delta (d_delta may be NULL; the sum is also stored
 *             to d_sum_out when that is not NULL - it must not alias d_x), then RMSNorm with d_norm_weight;
 *   behind    (silu_pair != 0, count == 2, N[0] == N[1]): d_y[0] = silu(linear0) * linear1, d_y[1] unused.
 * The fusions of QWenDecoder::forward / QWenMLP::forward (modeling_ds_qwen2.hpp:47-54,175-183) that cost a
 * launch each when run as separate operators. Returns W4A32_ENOTSUP when the shape does not fit the
 * single-launch kernel (the caller then runs the operators one by one). */
/* Zero-initialise the struct before filling it: fields added at its end (in_parts, out_parts) select other
 * forms of the call when they are not 0. */
typedef struct {
  const float* d_x;
  const float* d_delta;
  float* d_sum_out;
  const float* d_norm_weight;
  float norm_eps;
  int K;
  int count;
  const void* d_packed[4];
  int N[4];
  float* d_y[4];
  int silu_pair;
  int in_parts;   /* 0 or 1: a single row. 2 or 3: the row is given in that many partial rows, K floats apart, which
                     the launch adds up ((r0 + r1) + r2), clamped to the finite f32 range like every Linear
                     output, before it does anything else - at d_delta when
                     d_norm_weight is given (d_delta is then required), else at d_x. Not with silu_pair; for an
                     lm_head-sized Linear (N >= 32768) only as a single Linear with a norm (W4A32_ENOTSUP else). */
  int out_parts;  /* 0 or 1: d_y holds the Linears' outputs. > 1 (count == 1, no norm, no pair, in_parts <= 1;
                     must equal w4a32_decode_kparts(K, N[0])): the Linear's k range is dealt to that many workgroups
                     per tile row and d_y[0] receives [out_parts][N[0]] partial rows whose sum is the output (bias
                     included; the parts themselves are not clamped, a reader that adds them up clamps the sum),
                     for the next w4a32_decode_linear via in_parts. */
} w4a32_decode_linear_args;
int w4a32_decode_linear(const w4a32_decode_linear_args* args, void* stream);

/* Parts into which w4a32_decode_linear would split a [N][K] Linear's k range: 2 for a long K with few output
 * rows (down_proj, K = 8960, N = 1536: its 96 tile rows alone would leave 160 of 256 CUs idle), else 1 (no
 * split). 0 on an invalid shape. No counterpart in the reference, which runs a decode Linear as one task
 * (kai_linear.cpp:366-396). */
int w4a32_decode_kparts(int K, int N);

/* ---- operators of the engine's op-by-op path ------------------------------------------------
 * What the reference's model code dispatches one by one and the decoder runner below fuses away. They exist
 * so that a backend can offer every operator of mllm/Models/ds_qwen2/modeling_ds_qwen2_fa2_fp16.hpp:88-133
 * (activations [B, S, H, D], RoPE layout kBSHD, KV cache layout kBSHD_NO_REPEAT). n % 4 == 0. */

/* out = x / (1 + exp(-x)) (ArmSiLUOp, mllm/Backends/Arm/Ops/SiLUOp.cpp) and out = a * b (ArmMulOp,
 * mllm/Backends/Arm/Ops/ElewiseOps.cpp). SiLU followed by Mul equals w4a32_op_silu_mul bit for bit. */
int w4a32_op_silu(const float* d_x, float* d_out, size_t n, void* stream);
int w4a32_op_mul(const float* d_a, const float* d_b, float* d_out, size_t n, void* stream);

/* y[m][h][:] = RoPE of x[m][h][:] at position pos0 + m, rows [M][n_heads][head_dim] (normal_hf_rope_shd,
 * mllm/Backends/Arm/Kernels/rope.cpp, layout kBSHD); tables as w4a32_op_rope_table builds them, with
 * table_rows rows. d_y may be d_x. */
int w4a32_op_rope(const float* d_x, float* d_y, const float* d_sin, const float* d_cos, int M, int n_heads,
                  int head_dim, int pos0, int table_rows, void* stream);

/* Causal attention with K and V laid out [n_keys][n_kv_heads][head_dim] (the kBSHD_NO_REPEAT cache at batch
 * 1, mllm/Backends/Arm/Ops/KVCacheOp.cpp:74-88): query m at position pos0 + m sees keys 0..pos0 + m.
 * ArmFlashAttn2Op::forward, mllm/Backends/Arm/Ops/FlashAttention2Op.cpp:221-245. head_dim must be 128. */
int w4a32_op_attention_bshd(const float* d_q, const float* d_k, const float* d_v, float* d_out, int M,
                            int n_heads, int n_kv_heads, int head_dim, int n_keys, int pos0, void* stream);

/* C[M][N] = A[M][K] B[N][K]^T, dense f32 (MatMulOp with transpose_b, mllm/Backends/Arm/Ops/MatMulOp.cpp:131-167:
 * how the reference applies lm_head, modeling_ds_qwen2.hpp:209-213). K % 4 == 0. M <= 8 streams B once. */
int w4a32_op_matmul_f32_nt(const float* d_a, const float* d_b, float* d_c, int M, int N, int K, void* stream);

/* Element types of a dense (unquantised) operand. The reference's W4A32 quantizer configuration stores lm_head
 * and the three RMSNorm weights as Fp16 (scripts/QuantCfg/ds_qwen2/1.5B-W4A32-KAI.json:33-45). */
#define W4A32_DENSE_F32 1
#define W4A32_DENSE_F16 2

/* The same product with B [N][K] held as f32 or f16 (b_dtype = W4A32_DENSE_*): an f16 element widens to f32
 * exactly, every product and sum is f32. With K % 8 == 0 and M <= 8, B is streamed once and the f16 and the f32
 * form of the same values give identical bits. K % 4 == 0. */
int w4a32_op_matmul_nt(const float* d_a, const void* d_b, int b_dtype, float* d_c, int M, int N, int K,
                       void* stream);

/* d_out[i] = (float)d_in[i] for n IEEE half values (exact): Fp16 parameters of a model file are widened once at
 * load and the f32 operators run on the result. */
int w4a32_op_f16_to_f32(const void* d_in, float* d_out, size_t n, void* stream);

/* ---- decoder runner -------------------------------------------------------------------- */

typedef struct {
  int hidden, n_heads, n_kv_heads, head_dim, intermediate, n_layers, vocab;
  int max_seq;           /* KV cache capacity (the reference's max_cache_length) */
  int max_batch_tokens;  /* longest prompt chunk a prefill call may take */
  float rope_theta, rms_eps;
} w4a32_decoder_config;

/* Device pointers; W4 blobs as produced by w4a32_quant_pack_rhs ([N][K] = [out][in]). */
typedef struct {
  const void *q, *k, *v, *o, *gate, *up, *down;
  const float *attn_norm, *ffn_norm;
} w4a32_layer_weights;

/* Zero-initialise the struct before filling it (fields may be added at its end). */
typedef struct {
  const float* embedding;             /* [vocab][hidden] f32 */
  const float* final_norm;            /* [hidden] */
  const void* lm_head;                /* W4 blob [vocab][hidden]; may be NULL when lm_head_dense is given */
  const w4a32_layer_weights* layers;  /* HOST array of n_layers entries */
  /* lm_head as the reference applies it (a dense matmul with transpose_b, modeling_ds_qwen2.hpp:209-213):
   * [vocab][hidden] of lm_head_dense_dtype (W4A32_DENSE_F16 as the reference's quantizer stores it, or
   * W4A32_DENSE_F32). When not NULL it is used instead of lm_head; hidden % 8 == 0. */
  const void* lm_head_dense;
  int lm_head_dense_dtype;
} w4a32_decoder_weights;

/* Bytes of the decoder state (KV caches, activations, tables, counters), 256-byte aligned base. */
size_t w4a32_decoder_state_bytes(const w4a32_decoder_config* cfg);
/* Byte offsets inside the state, for inspection: 0 = position counter (int32), 1 = last logits
 * (f32 [vocab]), 2 = residual stream rows (f32 [max_batch_tokens][hidden]). */
size_t w4a32_decoder_state_offset(const w4a32_decoder_config* cfg, int which);

/* Builds the RoPE tables, clears the counters, position = 0. */
int w4a32_decoder_init(const w4a32_decoder_config* cfg, void* d_state, void* stream);

/* Runs n_tokens prompt tokens at positions pos0.. through the model (QWenForCausalLM::forward,
 * modeling_ds_qwen2.hpp:202-215), leaves the last row's logits in the state, the greedy next token in
 * *d_next_token and the position counter at pos0 + n_tokens. */
int w4a32_decoder_prefill(const w4a32_decoder_config* cfg, const w4a32_decoder_weights* w,
                          void* d_state, const int64_t* d_tokens, int n_tokens, int pos0,
                          int64_t* d_next_token, void* stream);

/* One greedy decode step at the state's current position (AutoLLM generate loop, AutoLLM.hpp:40-66):
 * reads *d_token_in, writes *d_token_out (may be the same address), advances the position. The launch
 * sequence does not depend on the position: capture it once, replay it per token. The caller keeps
 * the position below max_seq: the step itself cannot refuse (the position is device memory, and a replayed
 * graph never returns to the host). A step issued at position >= max_seq stays inside the cache - the
 * attention treats the position as max_seq - 1 and overwrites the last row - but its token is meaningless
 * and the counter keeps advancing; w4a32_decoder_prefill, whose pos0 is a host argument, returns W4A32_ESHAPE
 * when pos0 + n_tokens exceeds max_seq. */
int w4a32_decoder_step(const w4a32_decoder_config* cfg, const w4a32_decoder_weights* w, void* d_state,
                       const int64_t* d_token_in, int64_t* d_token_out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* W4A32_DECODER_H */
