// The f32 operators of a Qwen2-style decoder on MI355X behind the engine's operator interfaces, for model
// code that dispatches them one by one. They follow the layouts of the reference's flash-attention model
// variant (mllm/Models/ds_qwen2/modeling_ds_qwen2_fa2_fp16.hpp:88-133): activations [B, S, H, D], RoPE with
// layout kBSHD, KV cache with layout kBSHD_NO_REPEAT, FlashAttn2 on [B, S, H, D] operands - all in f32,
// batch 1. Reference counterparts: mllm/Backends/Arm/Ops/{View,RMSNorm,RoPE,KVCache,FlashAttention2,MatMul,
// SiLU,Elewise,LLMEmbeddingToken}Op(s).{hpp,cpp}; registered like mllm/Backends/Arm/ArmBackend.cpp:42-52.
//
// Each forward only enqueues kernels of libw4a32_hip.so (include/w4a32_decoder.h) on the backend's stream.
// The decoder runner (mllm/Models/ds_qwen2/HipQwen2.*) fuses most of these away; these classes are what a
// module tree of the reference's own kind lands on when its layers are moved to kHIP.
#pragma once

#include "mllm/Core/AOps/ElewiseOp.hpp"
#include "mllm/Core/AOps/FlashAttention2Op.hpp"
#include "mllm/Core/AOps/KVCacheOp.hpp"
#include "mllm/Core/AOps/LLMEmbeddingTokenOp.hpp"
#include "mllm/Core/AOps/MatMulOp.hpp"
#include "mllm/Core/AOps/RMSNormOp.hpp"
#include "mllm/Core/AOps/RoPEOp.hpp"
#include "mllm/Core/AOps/SiLUOp.hpp"
#include "mllm/Core/AOps/ViewOp.hpp"

namespace mllm::hip {

// Same memory, another shape: everything happens in ViewOp::reshape (mllm/Core/AOps/ViewOp.cpp:34-90).
class HipViewOp final : public ViewOp {
 public:
  explicit HipViewOp(const ViewOpCargo& cargo);
};

// y = x * (w * 1/sqrt(mean(x^2) + eps)) over the last dimension (ArmRMSNormOp::forward, RMSNormOp.cpp:20-76).
class HipRMSNormOp final : public RMSNormOp {
 public:
  explicit HipRMSNormOp(const RMSNormOpCargo& cargo);
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;  // uploads "<name>.weight"
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

// RoPE of [1, S, H, D] rows at positions cur_seq_cnt_.. (ArmRoPEOp::forward, RoPEOp.cpp:95-135, layout kBSHD);
// the position advances by S per call, as the reference's does. The sin / cos tables are built on the device
// once per (theta, max_position_embeddings, dims) and shared by all RoPE ops of the backend.
class HipRoPEOp final : public RoPEOp {
 public:
  explicit HipRoPEOp(const RoPEOpCargo& cargo);
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;

 private:
  void tables();
  Tensor sin_, cos_;
};

// Appends [1, S, H, D] to a device cache [1, limit, H, D] and returns the filled prefix [1, len + S, H, D]
// as a view of the cache (ArmKVCacheOp, KVCacheOp.cpp:74-88, 150-196, 208-214, layout kBSHD_NO_REPEAT).
// The cache grows by re_alloc_multiplier when it is full, keeping its contents.
class HipKVCacheOp final : public KVCacheOp {
 public:
  explicit HipKVCacheOp(const KVCacheOpCargo& cargo);
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  void setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;

 private:
  int32_t cur_kv_cache_limits_ = 0;
  int32_t cur_kv_cache_seq_len_ = 0;
};

// softmax(q k^T / sqrt(D) + causal mask) v on q [1, S, Hq, D] and k, v [1, S_kv, Hkv, D]; query i stands at
// position S_kv - S + i (ArmFlashAttn2Op::forward, FlashAttention2Op.cpp:221-245; f32 here, fp16 there).
class HipFlashAttn2Op final : public FlashAttn2Op {
 public:
  explicit HipFlashAttn2Op(const FlashAttn2OpCargo& cargo);
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

// C = A B^T for A [..., M, K] and a two-dimensional B [N, K] on the device, both f32: how the reference applies
// its dense lm_head (modeling_ds_qwen2.hpp:209-213; ArmMatMulOp::forward, MatMulOp.cpp:131-167).
class HipMatMulOp final : public MatMulOp {
 public:
  explicit HipMatMulOp(const MatMulOpCargo& cargo);
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

class HipSiLUOp final : public SiLUOp {
 public:
  explicit HipSiLUOp(const SiLUOpCargo& cargo);
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

// Same-shape element-wise sum and product (ArmAddOp / ArmMulOp, ElewiseOps.cpp).
class HipAddOp final : public AddOp {
 public:
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

class HipMulOp final : public MulOp {
 public:
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

// ids [B, S] (int64, on the host or on the device) -> rows of "<name>.weight" [vocab, hidden] on the device
// (ArmLLMEmbeddingTokenOp::forward, LLMEmbeddingTokenOp.cpp:24-50). Ids outside [0, vocab) are clamped.
class HipLLMEmbeddingTokenOp final : public LLMEmbeddingTokenOp {
 public:
  explicit HipLLMEmbeddingTokenOp(const LLMEmbeddingTokenOpCargo& cargo);
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;  // uploads the table
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

#define MLLM_HIP_OP_FACTORY(factory, op, type, cargo_t)                                  \
  class factory : public TypedOpFactory<type, cargo_t> {                                 \
   public:                                                                               \
    std::shared_ptr<BaseOp> createOpImpl(const cargo_t& cargo) override {                \
      return std::make_shared<op>(cargo);                                                \
    }                                                                                    \
  }

MLLM_HIP_OP_FACTORY(HipViewOpFactory, HipViewOp, OpType::kView, ViewOpCargo);
MLLM_HIP_OP_FACTORY(HipRMSNormOpFactory, HipRMSNormOp, OpType::kRMSNorm, RMSNormOpCargo);
MLLM_HIP_OP_FACTORY(HipRoPEOpFactory, HipRoPEOp, OpType::kRoPE, RoPEOpCargo);
MLLM_HIP_OP_FACTORY(HipKVCacheOpFactory, HipKVCacheOp, OpType::kKVCache, KVCacheOpCargo);
MLLM_HIP_OP_FACTORY(HipFlashAttn2OpFactory, HipFlashAttn2Op, OpType::kFlashAttention_2, FlashAttn2OpCargo);
MLLM_HIP_OP_FACTORY(HipMatMulOpFactory, HipMatMulOp, OpType::kMatMul, MatMulOpCargo);
MLLM_HIP_OP_FACTORY(HipSiLUOpFactory, HipSiLUOp, OpType::kSiLU, SiLUOpCargo);
MLLM_HIP_OP_FACTORY(HipLLMEmbeddingTokenOpFactory, HipLLMEmbeddingTokenOp, OpType::kLLMEmbeddingToken,
                    LLMEmbeddingTokenOpCargo);
#undef MLLM_HIP_OP_FACTORY

// the element-wise ops take no cargo in their constructors (mllm/Core/AOps/ElewiseOp.hpp:15-27)
class HipAddOpFactory : public TypedOpFactory<OpType::kAdd, AddOpCargo> {
 public:
  std::shared_ptr<BaseOp> createOpImpl(const AddOpCargo&) override { return std::make_shared<HipAddOp>(); }
};
class HipMulOpFactory : public TypedOpFactory<OpType::kMul, MulOpCargo> {
 public:
  std::shared_ptr<BaseOp> createOpImpl(const MulOpCargo&) override { return std::make_shared<HipMulOp>(); }
};

}  // namespace mllm::hip
