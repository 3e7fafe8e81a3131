#include "mllm/Models/ds_qwen2/HipQwen2.hpp"

#include <hip/hip_runtime_api.h>

#include <algorithm>

#include "mllm/Backends/HIP/HipBackend.hpp"
#include "mllm/Utils/Log.hpp"

namespace mllm::models {

namespace {

void check(int rc, const char* what) {
  if (rc != W4A32_OK) { MLLM_ERROR_EXIT(hip::kHipRuntimeError, "{} failed: {}", what, w4a32_error_string(rc)); }
}

void checkHip(hipError_t e, const char* what) {
  if (e != hipSuccess) { MLLM_ERROR_EXIT(hip::kHipRuntimeError, "{} failed: {}", what, hipGetErrorString(e)); }
}

}  // namespace

struct HipQWenForCausalLM::Impl {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  bool warmed = false;
  ~Impl() {
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
  }
};

HipQWenForCausalLM::HipQWenForCausalLM(const HipQWenConfig& cfg) : cfg_(cfg), impl_(new Impl) {
  dcfg_.hidden = cfg.hidden_size;
  dcfg_.n_heads = cfg.num_attention_heads;
  dcfg_.n_kv_heads = cfg.num_key_value_heads;
  dcfg_.head_dim = cfg.hidden_size / cfg.num_attention_heads;
  dcfg_.intermediate = cfg.intermediate_size;
  dcfg_.n_layers = cfg.num_hidden_layers;
  dcfg_.vocab = cfg.vocab_size;
  dcfg_.max_seq = cfg.max_cache_length;
  dcfg_.max_batch_tokens = std::min(cfg.max_prompt_chunk, cfg.max_cache_length);
  dcfg_.rope_theta = cfg.rope_theta;
  dcfg_.rms_eps = cfg.rms_norm_eps;
}

HipQWenForCausalLM::~HipQWenForCausalLM() = default;

void HipQWenForCausalLM::load(const std::shared_ptr<ParameterLoader>& ploader) {
  const int H = cfg_.hidden_size, D = dcfg_.head_dim;
  const int qd = cfg_.num_attention_heads * D, kvd = cfg_.num_key_value_heads * D;

  auto linear = [&](const std::string& name, int in, int out, bool bias) -> const void* {
    LinearOpCargo cargo;
    cargo.in_channels = in;
    cargo.out_channels = out;
    cargo.bias = bias;
    cargo.impl_type_ = cfg_.linear_impl_type;
    auto op = std::make_shared<hip::HipLinearOp>(cargo);
    op->setName(name);
    op->load(ploader);
    linears_.push_back(op);
    return op->weight().ptr<void>();
  };
  auto f32 = [&](const std::string& name, size_t numel) -> const float* {
    // Fp32, or Fp16 (the dtype the reference's W4A32 quantizer configuration gives the norm weights), widened once
    Tensor host((*ploader)[name]);
    if ((host.dtype() != kFp32 && host.dtype() != kFp16) || host.numel() != numel) {
      MLLM_ERROR_EXIT(kError, "{}: expected {} f32 or f16 values, got {} x {}", name, numel,
                      dataTypes2Str(host.dtype()), host.numel());
    }
    Tensor dev = hip::toDeviceF32(host);
    f32_params_.push_back(dev);
    return dev.ptr<float>();
  };

  layer_weights_.resize(cfg_.num_hidden_layers);
  for (int i = 0; i < cfg_.num_hidden_layers; ++i) {
    const std::string base = "model.layers." + std::to_string(i) + ".";
    auto& lw = layer_weights_[i];
    lw.attn_norm = f32(base + "input_layernorm.weight", H);
    lw.q = linear(base + "self_attn.q_proj", H, qd, true);
    lw.k = linear(base + "self_attn.k_proj", H, kvd, true);
    lw.v = linear(base + "self_attn.v_proj", H, kvd, true);
    lw.o = linear(base + "self_attn.o_proj", qd, H, false);
    lw.ffn_norm = f32(base + "post_attention_layernorm.weight", H);
    lw.gate = linear(base + "mlp.gate_proj", H, cfg_.intermediate_size, false);
    lw.up = linear(base + "mlp.up_proj", H, cfg_.intermediate_size, false);
    lw.down = linear(base + "mlp.down_proj", cfg_.intermediate_size, H, false);
  }
  weights_.embedding = f32("model.embed_tokens.weight", (size_t)cfg_.vocab_size * H);
  weights_.final_norm = f32("model.norm.weight", H);
  {
    Tensor head((*ploader)["lm_head.weight"]);
    const bool unquantised = head.dtype() == kFp32 || head.dtype() == kFp16;
    if (unquantised && !cfg_.lm_head_w4a32) {
      // the reference's form: x [S, D] times lm_head [V, D] transposed, on the tensor as the file holds it
      if (head.numel() != (size_t)cfg_.vocab_size * H) {
        MLLM_ERROR_EXIT(kError, "lm_head.weight: expected [{}, {}], got {} elements", cfg_.vocab_size, H, head.numel());
      }
      lm_head_dense_ = hip::toDevice(head);
      weights_.lm_head = nullptr;
      weights_.lm_head_dense = lm_head_dense_.ptr<void>();
      weights_.lm_head_dense_dtype = head.dtype() == kFp16 ? W4A32_DENSE_F16 : W4A32_DENSE_F32;
    } else {
      weights_.lm_head = linear("lm_head", H, cfg_.vocab_size, false);
    }
  }
  weights_.layers = layer_weights_.data();

  const size_t bytes = w4a32_decoder_state_bytes(&dcfg_);
  if (bytes == 0) {
    MLLM_ERROR_EXIT(kError, "unsupported decoder shape (head_dim must be 128, sizes multiples of 32)");
  }
  // A tensor dimension is an int32: the state (mostly the KV cache, 2 * layers * kv_heads * max_seq * 512
  // bytes) is counted in 8-byte elements, which reaches 16 GiB.
  const size_t words = (bytes + 7) / 8;
  if (words > 0x7FFFFFFFull) {
    MLLM_ERROR_EXIT(kMemory, "decoder state of {} bytes (max_cache_length {}) exceeds one tensor", bytes,
                    dcfg_.max_seq);
  }
  state_ = Tensor::empty({static_cast<int32_t>(words)}, kInt64, kHIP).alloc();
  token_ = Tensor::empty({1}, kInt64, kHIP).alloc();
  auto& hb = hip::currentHipBackend();
  check(w4a32_decoder_init(&dcfg_, state_.ptr<void>(), hb.stream()), "w4a32_decoder_init");
  hb.synchronize();
  position_ = 0;
}

void HipQWenForCausalLM::reset() { position_ = 0; }

int64_t HipQWenForCausalLM::prefill(const std::vector<int64_t>& tokens) {
  auto& hb = hip::currentHipBackend();
  auto stream = static_cast<hipStream_t>(hb.stream());
  if (tokens.empty()) { MLLM_ERROR_EXIT(kError, "prefill: empty prompt"); }
  if (position_ + (int)tokens.size() > dcfg_.max_seq) {
    MLLM_ERROR_EXIT(kError, "prefill: {} tokens at position {} exceed max_cache_length {}",
                    tokens.size(), position_, dcfg_.max_seq);
  }
  Tensor ids = Tensor::empty({static_cast<int32_t>(tokens.size())}, kInt64, kHIP).alloc();
  checkHip(hipMemcpyAsync(ids.ptr<void>(), tokens.data(), tokens.size() * sizeof(int64_t),
                          hipMemcpyHostToDevice, stream), "hipMemcpyAsync(tokens)");
  for (size_t done = 0; done < tokens.size();) {
    const int n = (int)std::min<size_t>(dcfg_.max_batch_tokens, tokens.size() - done);
    check(w4a32_decoder_prefill(&dcfg_, &weights_, state_.ptr<void>(), ids.ptr<int64_t>() + done, n,
                                position_, token_.ptr<int64_t>(), stream), "w4a32_decoder_prefill");
    position_ += n;
    done += n;
  }
  int64_t next = 0;
  checkHip(hipMemcpyAsync(&next, token_.ptr<void>(), sizeof(next), hipMemcpyDeviceToHost, stream),
           "hipMemcpyAsync(token)");
  hb.synchronize();  // ids is released on return
  return next;
}

int64_t HipQWenForCausalLM::step() {
  auto& hb = hip::currentHipBackend();
  auto stream = static_cast<hipStream_t>(hb.stream());
  if (position_ >= dcfg_.max_seq) {
    MLLM_ERROR_EXIT(kError, "step: the cache (max_cache_length {}) is full", dcfg_.max_seq);
  }
  if (!impl_->warmed) {
    // The very first step runs eagerly: it brings the decode kernels' code objects in, which must
    // not happen inside a stream capture.
    check(w4a32_decoder_step(&dcfg_, &weights_, state_.ptr<void>(), token_.ptr<int64_t>(),
                             token_.ptr<int64_t>(), stream), "w4a32_decoder_step");
    impl_->warmed = true;
  } else {
    if (!impl_->exec) {
      // One step's launch sequence does not depend on the position (it lives in device memory), so
      // it is recorded once. The capture executes nothing.
      checkHip(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
      const int rc = w4a32_decoder_step(&dcfg_, &weights_, state_.ptr<void>(), token_.ptr<int64_t>(),
                                        token_.ptr<int64_t>(), stream);
      checkHip(hipStreamEndCapture(stream, &impl_->graph), "hipStreamEndCapture");
      check(rc, "w4a32_decoder_step");
      checkHip(hipGraphInstantiate(&impl_->exec, impl_->graph, nullptr, nullptr, 0), "hipGraphInstantiate");
    }
    checkHip(hipGraphLaunch(impl_->exec, stream), "hipGraphLaunch");
  }
  int64_t next = 0;
  checkHip(hipMemcpyAsync(&next, token_.ptr<void>(), sizeof(next), hipMemcpyDeviceToHost, stream),
           "hipMemcpyAsync(token)");
  hb.synchronize();
  ++position_;
  return next;
}

std::vector<int64_t> HipQWenForCausalLM::generate(const std::vector<int64_t>& prompt, int32_t max_length) {
  std::vector<int64_t> out;
  int64_t tok = prefill(prompt);
  out.push_back(tok);
  while (position_ < std::min(max_length, dcfg_.max_seq) && tok != cfg_.eos_token_id) {
    tok = step();
    out.push_back(tok);
  }
  return out;
}

std::vector<float> HipQWenForCausalLM::lastLogits() const {
  auto& hb = hip::currentHipBackend();
  std::vector<float> logits(dcfg_.vocab);
  const size_t off = w4a32_decoder_state_offset(&dcfg_, 1);
  checkHip(hipMemcpyAsync(logits.data(), state_.ptr<uint8_t>() + off, logits.size() * sizeof(float),
                          hipMemcpyDeviceToHost, static_cast<hipStream_t>(hb.stream())),
           "hipMemcpyAsync(logits)");
  hb.synchronize();
  return logits;
}

}  // namespace mllm::models
