// DeepSeek-Distill-Qwen2 / Qwen2 decoder on MI355X: the module tree of the reference
// (mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:28-216) and its generation loop
// (mllm/Models/AutoLLM.hpp:40-105) collapsed into one object that loads the same parameter names
// from a .mllm file and runs on the device-side decoder runner (include/w4a32_decoder.h).
//
// Parameter names, as the reference's modules register them:
//   model.embed_tokens.weight                       f32 [vocab, hidden]
//   model.layers.<i>.input_layernorm.weight         f32 [hidden]
//   model.layers.<i>.self_attn.{q,k,v}_proj.{weight,bias}, o_proj.weight
//   model.layers.<i>.post_attention_layernorm.weight
//   model.layers.<i>.mlp.{gate,up,down}_proj.weight
//   model.norm.weight, lm_head.weight
// Linear weights may be f32 / f16 [out, in] (quantised on load), this build's int8 W4 file blob or the Arm
// quantizer's blob, as HipLinearOp::load accepts them. The norm weights and the embedding may be Fp32 or Fp16
// (widened once at load). lm_head.weight is applied as the reference applies it, a dense matmul with
// transpose_b (modeling_ds_qwen2.hpp:209-213), on the tensor as the file holds it: Fp16 [vocab, hidden] (what
// the reference's W4A32 quantizer configuration writes, scripts/QuantCfg/ds_qwen2/1.5B-W4A32-KAI.json:33-45)
// or Fp32. With HipQWenConfig::lm_head_w4a32 it is quantised to a W4A32 Linear instead (the benchmark's
// lm_head shape); an int8 W4 blob under that name is always a W4A32 Linear.
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "mllm/Backends/HIP/Ops/LinearOp.hpp"
#include "mllm/Core/Tensor.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "w4a32_decoder.h"

namespace mllm::models {

// The fields of the reference's QWenConfig (configuration_ds_qwen2.hpp:18-90) this model reads, under the
// same names and with the same defaults; a struct of its own name so that it can live beside the reference's
// (whose constructor wants a JSON file) in one program.
struct HipQWenConfig {
  int32_t num_attention_heads = 12;
  int32_t num_hidden_layers = 28;
  int32_t num_key_value_heads = 2;
  int32_t hidden_size = 1536;
  int32_t intermediate_size = 8960;
  float rope_theta = 10000.f;
  int32_t max_position_embeddings = 131072;
  float rms_norm_eps = 1e-06;
  int32_t vocab_size = 151936;
  int32_t max_cache_length = 1024;
  int64_t eos_token_id = 151643;
  LinearOpImplType linear_impl_type =
      LinearOpImplType::kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p4x8_8x4x32;
  int32_t max_prompt_chunk = 512;  // longest prompt slice one prefill call takes (not in the reference)
  bool lm_head_w4a32 = false;      // quantise an Fp32 / Fp16 lm_head to W4A32 instead of the dense matmul (not in the reference)
};

class HipQWenForCausalLM {
 public:
  explicit HipQWenForCausalLM(const HipQWenConfig& cfg);
  ~HipQWenForCausalLM();
  HipQWenForCausalLM(const HipQWenForCausalLM&) = delete;
  HipQWenForCausalLM& operator=(const HipQWenForCausalLM&) = delete;

  // Module::load: uploads / quantises every parameter, allocates the decoder state.
  void load(const std::shared_ptr<ParameterLoader>& ploader);

  // Greedy generation (AutoLLM::generate with greedy search): feeds the prompt, then decodes until
  // max_length tokens exist or eos is produced. Returns the generated tokens (prompt excluded).
  // The decode step is captured into a HIP graph on first use and replayed per token.
  std::vector<int64_t> generate(const std::vector<int64_t>& prompt, int32_t max_length);

  // The pieces generate() is made of, for callers that keep their own loop.
  int64_t prefill(const std::vector<int64_t>& tokens);  // appends at the current position
  int64_t step();                                       // consumes the last produced token
  void reset();                                         // position 0 (the cache is overwritten)
  [[nodiscard]] int32_t position() const { return position_; }
  [[nodiscard]] std::vector<float> lastLogits() const;  // device -> host copy of [vocab]

 private:
  struct Impl;
  HipQWenConfig cfg_;
  w4a32_decoder_config dcfg_{};
  std::vector<std::shared_ptr<hip::HipLinearOp>> linears_;  // keep the device blobs alive
  std::vector<Tensor> f32_params_;
  Tensor lm_head_dense_;  // [vocab, hidden] f16 or f32 on the device, when lm_head is applied densely
  std::vector<w4a32_layer_weights> layer_weights_;
  w4a32_decoder_weights weights_{};
  Tensor state_, token_;
  int32_t position_ = 0;
  std::unique_ptr<Impl> impl_;  // the captured graph
};

}  // namespace mllm::models
