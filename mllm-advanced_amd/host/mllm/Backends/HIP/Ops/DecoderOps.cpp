#include "mllm/Backends/HIP/Ops/DecoderOps.hpp"

#include <hip/hip_runtime_api.h>

#include "mllm/Backends/HIP/HipBackend.hpp"
#include "mllm/Engine/Context.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "mllm/Utils/Log.hpp"
#include "w4a32_decoder.h"

namespace mllm::hip {

namespace {

void check(int rc, const char* what) {
  if (rc != W4A32_OK) { MLLM_ERROR_EXIT(kHipRuntimeError, "{} failed: {}", what, w4a32_error_string(rc)); }
}

void checkHip(hipError_t e, const char* what) {
  if (e != hipSuccess) { MLLM_ERROR_EXIT(kHipRuntimeError, "{} failed: {}", what, hipGetErrorString(e)); }
}

// what every operator here asks of an operand: f32, on this device
void wantF32OnHip(const Tensor& t, const std::string& op, const char* which) {
  if (t.device() != kHIP || t.dtype() != kFp32) {
    MLLM_ERROR_EXIT(kError, "{}: {} must be an f32 tensor on the HIP device", op, which);
  }
}

}  // namespace

HipViewOp::HipViewOp(const ViewOpCargo& cargo) : ViewOp(cargo) {}

// ---------------------------------------------------------------------------- RMSNorm
HipRMSNormOp::HipRMSNormOp(const RMSNormOpCargo& cargo) : RMSNormOp(cargo) {}

void HipRMSNormOp::load(const std::shared_ptr<ParameterLoader>& ploader) {
  RMSNormOp::load(ploader);
  // Fp32, or Fp16 as the reference's W4A32 quantizer configuration stores it: widened once, here
  if (weight_.device() != kHIP) weight_ = toDeviceF32(weight_);
  if (weight_.dtype() != kFp32) { MLLM_ERROR_EXIT(kError, "{}.weight must be f32 or f16", name()); }
}

void HipRMSNormOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& x = inputs[0];
  wantF32OnHip(x, name(), "input");
  if (weight_.isNil() || weight_.device() != kHIP) { MLLM_ERROR_EXIT(kError, "{}: forward before load", name()); }
  if (cargo_.add_unit_offset) { MLLM_ERROR_EXIT(kError, "{}: add_unit_offset is not implemented on HIP", name()); }
  const auto shape = x.shape();
  const int D = shape[shape.size() - 1];
  MLLM_RT_ASSERT_EQ(static_cast<size_t>(D), weight_.numel());
  const int M = static_cast<int>(x.numel() / static_cast<size_t>(D));
  check(w4a32_op_rmsnorm(x.ptr<float>(), nullptr, weight_.ptr<float>(), M, D, cargo_.epsilon, nullptr,
                         outputs[0].ptr<float>(), currentHipBackend().stream()),
        "w4a32_op_rmsnorm");
}

// ---------------------------------------------------------------------------- RoPE
HipRoPEOp::HipRoPEOp(const RoPEOpCargo& cargo) : RoPEOp(cargo) {}

void HipRoPEOp::tables() {
  if (!sin_.isNil()) return;
  if (cargo_.type != RoPETypes::kLlama2) { MLLM_ERROR_EXIT(kError, "{}: unsupported rope type", name()); }
  currentHipBackend().ropeTables(cargo_.theta, cargo_.max_position_embeddings, cargo_.dims, &sin_, &cos_);
}

void HipRoPEOp::load(const std::shared_ptr<ParameterLoader>& ploader) { tables(); }

void HipRoPEOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& x = inputs[0];
  wantF32OnHip(x, name(), "input");
  if (cargo_.layout_type != RoPEOpCargo::kBSHD) {
    MLLM_ERROR_EXIT(kError, "{}: the HIP backend rotates [B, S, H, D] rows (layout kBSHD) only", name());
  }
  const auto shape = x.shape();
  MLLM_RT_ASSERT_EQ(shape.size(), 4);
  MLLM_RT_ASSERT_EQ(shape[0], 1);
  MLLM_RT_ASSERT_EQ(shape[3], cargo_.dims);
  tables();
  const int S = shape[1], H = shape[2], D = shape[3];
  if (cur_seq_cnt_ + S > cargo_.max_position_embeddings) {
    MLLM_ERROR_EXIT(kError, "{}: position {} exceeds max_position_embeddings {}", name(), cur_seq_cnt_ + S,
                    cargo_.max_position_embeddings);
  }
  check(w4a32_op_rope(x.ptr<float>(), outputs[0].ptr<float>(), sin_.ptr<float>(), cos_.ptr<float>(), S, H, D,
                      cur_seq_cnt_, cargo_.max_position_embeddings, currentHipBackend().stream()),
        "w4a32_op_rope");
  cur_seq_cnt_ += S;
}

// ---------------------------------------------------------------------------- KV cache
HipKVCacheOp::HipKVCacheOp(const KVCacheOpCargo& cargo) : KVCacheOp(cargo) {
  cur_kv_cache_limits_ = cargo_.pre_alloc_seq_len;
}

void HipKVCacheOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  MLLM_RT_ASSERT_EQ(inputs.size(), 1);
  wantF32OnHip(inputs[0], name(), "input");
  if (cargo_.layout_type != KVCacheOpCargo::kBSHD_NO_REPEAT || cargo_.cached_elements_dtype != kFp32) {
    MLLM_ERROR_EXIT(kError, "{}: the HIP backend keeps an f32 cache in layout kBSHD_NO_REPEAT only", name());
  }
  const auto shape = inputs[0].shape();  // [B, S, H, D]
  MLLM_RT_ASSERT_EQ(shape.size(), 4);
  MLLM_RT_ASSERT_EQ(shape[0], 1);
  MLLM_RT_ASSERT_EQ(shape[2], cargo_.heads_num);
  MLLM_RT_ASSERT_EQ(shape[3], cargo_.dim_per_head);
  const int S = shape[1];
  const size_t row = static_cast<size_t>(cargo_.heads_num) * cargo_.dim_per_head;  // floats per position
  int32_t limits = cur_kv_cache_limits_;
  while (cur_kv_cache_seq_len_ + S > limits) limits *= cargo_.re_alloc_multiplier;
  if (cache_.isNil() || limits != cur_kv_cache_limits_) {
    Tensor grown = Tensor::empty({1, limits, cargo_.heads_num, cargo_.dim_per_head}, kFp32, kHIP).alloc();
    if (!cache_.isNil() && cur_kv_cache_seq_len_ > 0) {
      MLLM_WARN("Trying to expand KVCache from {} to {}", cur_kv_cache_limits_, limits);
      // positions are the outermost dimension at batch 1: the filled prefix is one contiguous range
      checkHip(hipMemcpyAsync(grown.ptr<char>(), cache_.ptr<char>(), cur_kv_cache_seq_len_ * row * sizeof(float),
                              hipMemcpyDeviceToDevice, static_cast<hipStream_t>(currentHipBackend().stream())),
               "hipMemcpyAsync(KV cache)");
    }
    cache_ = grown;  // the old block returns to the memory manager; the stream orders its reuse behind the copy
    cur_kv_cache_limits_ = limits;
  }
}

void HipKVCacheOp::setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const int S = inputs[0].shape()[1];
  outputs.emplace_back(Tensor(TensorViewImpl::create(
      0, {1, cur_kv_cache_seq_len_ + S, cargo_.heads_num, cargo_.dim_per_head}, cache_.impl()->storage())));
}

void HipKVCacheOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const int S = inputs[0].shape()[1];
  const size_t row = static_cast<size_t>(cargo_.heads_num) * cargo_.dim_per_head;
  checkHip(hipMemcpyAsync(cache_.ptr<float>() + cur_kv_cache_seq_len_ * row, inputs[0].ptr<float>(),
                          S * row * sizeof(float), hipMemcpyDeviceToDevice,
                          static_cast<hipStream_t>(currentHipBackend().stream())),
           "hipMemcpyAsync(KV append)");
  cur_kv_cache_seq_len_ += S;
}

// ---------------------------------------------------------------------------- attention
HipFlashAttn2Op::HipFlashAttn2Op(const FlashAttn2OpCargo& cargo) : FlashAttn2Op(cargo) {}

void HipFlashAttn2Op::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  MLLM_RT_ASSERT_EQ(inputs.size(), 3);
  wantF32OnHip(inputs[0], name(), "q");
  wantF32OnHip(inputs[1], name(), "k");
  wantF32OnHip(inputs[2], name(), "v");
  if (!cargo_.causal_mask) { MLLM_ERROR_EXIT(kError, "{}: attention without the causal mask is not implemented on HIP", name()); }
  const auto qs = inputs[0].shape(), ks = inputs[1].shape();
  MLLM_RT_ASSERT_EQ(qs.size(), 4);
  MLLM_RT_ASSERT_EQ(qs[0], 1);
  MLLM_RT_ASSERT_EQ(qs[2], cargo_.q_head);
  MLLM_RT_ASSERT_EQ(ks[2], cargo_.kv_head);
  MLLM_RT_ASSERT_EQ(qs[3], cargo_.D);
  const int S = qs[1], S_kv = ks[1];
  check(w4a32_op_attention_bshd(inputs[0].ptr<float>(), inputs[1].ptr<float>(), inputs[2].ptr<float>(),
                                outputs[0].ptr<float>(), S, cargo_.q_head, cargo_.kv_head, cargo_.D, S_kv,
                                S_kv - S, currentHipBackend().stream()),
        "w4a32_op_attention_bshd");
}

// ---------------------------------------------------------------------------- dense matmul
HipMatMulOp::HipMatMulOp(const MatMulOpCargo& cargo) : MatMulOp(cargo) {}

void HipMatMulOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  wantF32OnHip(inputs[0], name(), "A");
  // B: f32, or f16 as the reference's quantizer stores lm_head (its elements widen exactly inside the kernel)
  const auto& B = inputs[1];
  if (B.device() != kHIP || (B.dtype() != kFp32 && B.dtype() != kFp16)) {
    MLLM_ERROR_EXIT(kError, "{}: B must be an f32 or f16 tensor on the HIP device (move a host parameter there "
                    "once, with hip::toDevice)", name());
  }
  const auto bs = inputs[1].shape();
  if (cargo_.transpose_a || !cargo_.transpose_b || bs.size() != 2) {
    MLLM_ERROR_EXIT(kError, "{}: the HIP backend implements A [.., M, K] x B [N, K]^T (transpose_b) only", name());
  }
  const int N = bs[0], K = bs[1];
  const int M = static_cast<int>(inputs[0].numel() / static_cast<size_t>(K));
  check(w4a32_op_matmul_nt(inputs[0].ptr<float>(), B.ptr<void>(), B.dtype() == kFp16 ? W4A32_DENSE_F16 : W4A32_DENSE_F32,
                           outputs[0].ptr<float>(), M, N, K, currentHipBackend().stream()),
        "w4a32_op_matmul_nt");
}

// ---------------------------------------------------------------------------- element-wise
HipSiLUOp::HipSiLUOp(const SiLUOpCargo& cargo) : SiLUOp(cargo) {}

void HipSiLUOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  wantF32OnHip(inputs[0], name(), "input");
  check(w4a32_op_silu(inputs[0].ptr<float>(), outputs[0].ptr<float>(), inputs[0].numel(),
                      currentHipBackend().stream()),
        "w4a32_op_silu");
}

void HipAddOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  wantF32OnHip(inputs[0], "Add", "input 0");
  wantF32OnHip(inputs[1], "Add", "input 1");
  MLLM_RT_ASSERT_EQ(inputs[0].numel(), inputs[1].numel());  // no broadcast
  check(w4a32_op_add(inputs[0].ptr<float>(), inputs[1].ptr<float>(), outputs[0].ptr<float>(), inputs[0].numel(),
                     currentHipBackend().stream()),
        "w4a32_op_add");
}

void HipMulOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  wantF32OnHip(inputs[0], "Mul", "input 0");
  wantF32OnHip(inputs[1], "Mul", "input 1");
  MLLM_RT_ASSERT_EQ(inputs[0].numel(), inputs[1].numel());  // no broadcast
  check(w4a32_op_mul(inputs[0].ptr<float>(), inputs[1].ptr<float>(), outputs[0].ptr<float>(), inputs[0].numel(),
                     currentHipBackend().stream()),
        "w4a32_op_mul");
}

// ---------------------------------------------------------------------------- embedding
HipLLMEmbeddingTokenOp::HipLLMEmbeddingTokenOp(const LLMEmbeddingTokenOpCargo& cargo)
    : LLMEmbeddingTokenOp(cargo) {}

void HipLLMEmbeddingTokenOp::load(const std::shared_ptr<ParameterLoader>& ploader) {
  LLMEmbeddingTokenOp::load(ploader);
  if ((weight_.dtype() != kFp32 && weight_.dtype() != kFp16) ||
      weight_.numel() != static_cast<size_t>(cargo_.vocab_size) * cargo_.hidden_size) {
    MLLM_ERROR_EXIT(kError, "{}.weight must be f32 or f16 [{}, {}]", name(), cargo_.vocab_size, cargo_.hidden_size);
  }
  if (weight_.device() != kHIP) weight_ = toDeviceF32(weight_);
}

void HipLLMEmbeddingTokenOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto shape = inputs[0].shape();  // [batch, seq]; the ids may still be on the host
  MLLM_RT_ASSERT_EQ(shape.size(), 2);
  outputs.emplace_back(Tensor::empty({shape[0], shape[1], cargo_.hidden_size}, kFp32, kHIP));
}

void HipLLMEmbeddingTokenOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  if (weight_.isNil() || weight_.device() != kHIP) { MLLM_ERROR_EXIT(kError, "{}: forward before load", name()); }
  if (inputs[0].dtype() != kInt64) { MLLM_ERROR_EXIT(kError, "{}: token ids must be int64", name()); }
  Tensor ids = inputs[0].device() == kHIP ? inputs[0] : toDevice(inputs[0]);
  check(w4a32_op_embedding(ids.ptr<int64_t>(), weight_.ptr<float>(), static_cast<int>(ids.numel()),
                           cargo_.hidden_size, cargo_.vocab_size, outputs[0].ptr<float>(),
                           currentHipBackend().stream()),
        "w4a32_op_embedding");
}

}  // namespace mllm::hip
