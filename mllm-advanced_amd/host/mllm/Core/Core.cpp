// Tensor, BaseOp::setup and the device-independent halves of the operators.
#include <numeric>

#include "mllm/Core/AOps/LinearOp.hpp"
#include "mllm/Core/Tensor.hpp"
#include "mllm/Engine/Context.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "mllm/Utils/Log.hpp"

namespace mllm {

// ---------------------------------------------------------------------------- tensor
TensorStorage::~TensorStorage() {
  // kParams storage aliases a mapped file and is never freed here; the rest goes back to the memory manager
  // (reference: mllm/Core/TensorImpl.cpp:17-34).
  if (ptr_ && (mem_type_ == kNormal || mem_type_ == kGlobal)) MllmEngineCtx::instance().mem()->free(this);
}

std::shared_ptr<TensorStorage> TensorStorage::create(const std::vector<int32_t>& shape, DataTypes dtype,
                                                     DeviceTypes device) {
  auto ret = std::make_shared<TensorStorage>();
  ret->dtype_ = dtype;
  ret->device_ = device;
  size_t cnt = 1;
  for (int32_t d : shape) cnt *= static_cast<size_t>(d);
  ret->size_ = cnt * dataTypeSize(dtype);
  ret->custom_32bit_uuid_ = MllmEngineCtx::instance().getUUID();
  return ret;
}

size_t TensorViewImpl::numel() const {
  size_t n = 1;
  for (int32_t d : shape_) n *= static_cast<size_t>(d);
  return n;
}

std::vector<int32_t> TensorViewImpl::stride() const {
  std::vector<int32_t> st(shape_.size(), 1);
  for (int i = static_cast<int>(shape_.size()) - 2; i >= 0; --i) st[i] = st[i + 1] * shape_[i + 1];
  return st;
}

std::shared_ptr<TensorViewImpl> TensorViewImpl::create(const std::vector<int32_t>& shape,
                                                       const std::shared_ptr<TensorStorage>& storage) {
  return create(0, shape, storage);
}

std::shared_ptr<TensorViewImpl> TensorViewImpl::create(int32_t storage_offset, const std::vector<int32_t>& shape,
                                                       const std::shared_ptr<TensorStorage>& storage) {
  auto v = std::make_shared<TensorViewImpl>();
  v->storage_offset_ = storage_offset;
  v->shape_ = shape;
  v->storage_ = storage;
  return v;
}

Tensor Tensor::empty(const std::vector<int32_t>& shape, DataTypes dtype, DeviceTypes device) {
  return Tensor(TensorViewImpl::create(shape, TensorStorage::create(shape, dtype, device)));
}

Tensor& Tensor::alloc() {
  if (!impl_->storage()->ptr_) MllmEngineCtx::instance().mem()->alloc(impl_->storage());
  return *this;
}

Tensor& Tensor::setName(const std::string& name) {
  impl_->storage()->name_ = name;
  return *this;
}

Tensor& Tensor::setMemType(TensorMemTypes mem_type) {
  impl_->storage()->mem_type_ = mem_type;
  return *this;
}

Tensor Tensor::view(const std::vector<int>& indicies) {
  ViewOpCargo cargo;
  cargo.to_shape_ = indicies;
  return MllmEngineCtx::instance().dispatch(OpType::kView, cargo, {*this})[0];
}

// ---------------------------------------------------------------------------- operators
const char* opType2Str(OpType type) {
  switch (type) {
    case OpType::kAdd: return "kAdd";
    case OpType::kMul: return "kMul";
    case OpType::kMatMul: return "kMatMul";
    case OpType::kLLMEmbeddingToken: return "kLLMEmbeddingToken";
    case OpType::kLinear: return "kLinear";
    case OpType::kRoPE: return "kRoPE";
    case OpType::kRMSNorm: return "kRMSNorm";
    case OpType::kSiLU: return "kSiLU";
    case OpType::kKVCache: return "kKVCache";
    case OpType::kD2H: return "kD2H";
    case OpType::kView: return "kView";
    case OpType::kFlashAttention_2: return "kFlashAttention_2";
    default: return "Unknown";
  }
}

void BaseOp::setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  (void)inputs;
  for (auto& o : outputs) {
    if (!o.impl()->storage()->ptr_) o.alloc();
  }
}

namespace {
// the shape / type / device of input 0: what most operators' reshape produces
void likeInput0(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  outputs.emplace_back(Tensor::empty(inputs[0].shape(), inputs[0].dtype(), inputs[0].device()));
}
}  // namespace

LinearOpImplType LinearOpCargo::parseLinearOpImplTypeStr(const std::string& type_str) {
  using T = LinearOpImplType;
  static const std::string w4 = "KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk:";
  static const std::string w4a16 = "KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk:";
  static const std::pair<std::string, T> table[] = {
      {"Default", T::kDefault},
      {"Kai_Start", T::kKai_Start},
      {"KaiLinear_fp16_fp16_fp16p_mxk_kxn", T::kKaiLinear_fp16_fp16_fp16p_mxk_kxn},
      {w4 + "qai8dxp1x8_qsi4c32p4x8_1x4x32",
       T::kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x8_qsi4c32p4x8_1x4x32},
      {w4 + "qai8dxp1x8_qsi4c32p8x8_1x8x32",
       T::kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x8_qsi4c32p8x8_1x8x32},
      {w4 + "qai8dxp4x8_qsi4c32p4x8_8x4x32",
       T::kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p4x8_8x4x32},
      {w4 + "qai8dxp4x8_qsi4c32p4x8_16x4x32",
       T::kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p4x8_16x4x32},
      {w4 + "qai8dxp4x8_qsi4c32p8x8_4x8x32",
       T::kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p8x8_4x8x32},
      {w4 + "qai8dxp1x4_qsi4c32p4x4_1x4",
       T::kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x4_qsi4c32p4x4_1x4},
      {w4a16 + "qsi8d32p1x8_qai4c32p4x8_1x4",
       T::KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p1x8_qai4c32p4x8_1x4},
      {w4a16 + "qsi8d32p4x4_qai4c32p4x4_8x4",
       T::KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p4x4_qai4c32p4x4_8x4},
      {w4a16 + "qsi8d32p4x8_qai4c32p4x8_8x4_i8mm",
       T::KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p4x8_qai4c32p4x8_8x4_i8mm},
      {"Kai_End", T::kKai_End},
  };
  for (const auto& e : table) {
    if (e.first == type_str) return e.second;
  }
  MLLM_WARN("Can't parse Linear Impl Type: {}. Fallback to default impl.", type_str);
  return T::kDefault;
}

LinearOp::LinearOp(const LinearOpCargo& cargo) : BaseOp(OpType::kLinear), cargo_(cargo) {}

void LinearOp::load(const std::shared_ptr<ParameterLoader>& ploader) {
  weight_ = Tensor((*ploader)[name() + ".weight"]);
  if (cargo_.bias) bias_ = Tensor((*ploader)[name() + ".bias"]);
}

void LinearOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& i = inputs[0];
  auto o_shape = i.shape();
  MLLM_RT_ASSERT_EQ(o_shape[o_shape.size() - 1], cargo_.in_channels);
  o_shape[o_shape.size() - 1] = cargo_.out_channels;
  outputs.emplace_back(Tensor::empty(o_shape, i.dtype(), i.device()));
}

LinearOp::params_t LinearOp::params() {
  params_t ret;
  ret.insert({name() + ".weight", weight_});
  if (cargo_.bias) ret.insert({name() + ".bias", bias_});
  return ret;
}

D2HOp::D2HOp(const D2HOpCargo& cargo) : BaseOp(OpType::kD2H), cargo_(cargo) {}

void D2HOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  outputs.emplace_back(Tensor::empty(inputs[0].shape(), inputs[0].dtype(), cargo_.to_device_type));
}

ViewOp::ViewOp(const ViewOpCargo& cargo) : BaseOp(OpType::kView), cargo_(cargo) {}

void ViewOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& it = inputs[0];
  std::vector<int32_t> shape = cargo_.to_shape_;
  int infer = -1;
  size_t known = 1;
  for (size_t i = 0; i < shape.size(); ++i) {
    if (shape[i] == -1) {
      MLLM_RT_ASSERT(infer == -1);  // one dimension at most is inferred
      infer = static_cast<int>(i);
    } else {
      known *= static_cast<size_t>(shape[i]);
    }
  }
  if (infer != -1) {
    MLLM_RT_ASSERT(known != 0);
    MLLM_RT_ASSERT(it.numel() % known == 0);
    shape[infer] = static_cast<int32_t>(it.numel() / known);
    known *= static_cast<size_t>(shape[infer]);
  }
  MLLM_RT_ASSERT_EQ(it.numel(), known);
  outputs.emplace_back(Tensor(TensorViewImpl::create(it.impl()->storageOffset(), shape, it.impl()->storage())));
}

void ViewOp::setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  // nothing to allocate: the output is the input's memory
}

RMSNormOp::RMSNormOp(const RMSNormOpCargo& cargo) : BaseOp(OpType::kRMSNorm), cargo_(cargo) {}

void RMSNormOp::load(const std::shared_ptr<ParameterLoader>& ploader) {
  weight_ = Tensor((*ploader)[name() + ".weight"]);
}

void RMSNormOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  likeInput0(inputs, outputs);
}

RMSNormOp::params_t RMSNormOp::params() {
  params_t ret;
  ret.insert({name() + ".weight", weight_});
  return ret;
}

RoPEOp::RoPEOp(const RoPEOpCargo& cargo) : BaseOp(OpType::kRoPE), cargo_(cargo) {}

void RoPEOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  likeInput0(inputs, outputs);
}

KVCacheOp::KVCacheOp(const KVCacheOpCargo& cargo) : BaseOp(OpType::kKVCache), cargo_(cargo) {}

FlashAttn2Op::FlashAttn2Op(const FlashAttn2OpCargo& cargo) : BaseOp(OpType::kFlashAttention_2), cargo_(cargo) {}

void FlashAttn2Op::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  likeInput0(inputs, outputs);  // the query's shape
}

MatMulOp::MatMulOp(const MatMulOpCargo& cargo) : BaseOp(OpType::kMatMul), cargo_(cargo) {}

void MatMulOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto a = inputs[0].shape(), b = inputs[1].shape();
  MLLM_RT_ASSERT(a.size() >= 2 && b.size() >= 2);
  std::vector<int32_t> c(a.begin(), a.end() - 2);
  if (!cargo_.transpose_a && !cargo_.transpose_b) {  // [M, K] x [K, N]
    MLLM_RT_ASSERT_EQ(a[a.size() - 1], b[b.size() - 2]);
    c.push_back(a[a.size() - 2]);
    c.push_back(b[b.size() - 1]);
  } else if (!cargo_.transpose_a && cargo_.transpose_b) {  // [M, K] x [N, K]
    MLLM_RT_ASSERT_EQ(a[a.size() - 1], b[b.size() - 1]);
    c.push_back(a[a.size() - 2]);
    c.push_back(b[b.size() - 2]);
  } else {
    NYI("MatMulOp::reshape with transpose_a={} and transpose_b={} is not supported yet", cargo_.transpose_a,
        cargo_.transpose_b);
  }
  outputs.emplace_back(Tensor::empty(c, inputs[0].dtype(), inputs[0].device()));
}

SiLUOp::SiLUOp(const SiLUOpCargo& cargo) : BaseOp(OpType::kSiLU), cargo_(cargo) {}

void SiLUOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  likeInput0(inputs, outputs);
}

AddOp::AddOp() : BaseOp(OpType::kAdd) {}
void AddOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) { likeInput0(inputs, outputs); }

MulOp::MulOp() : BaseOp(OpType::kAdd) {}  // sic: the reference's macro gives every element-wise op kAdd
void MulOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) { likeInput0(inputs, outputs); }

LLMEmbeddingTokenOp::LLMEmbeddingTokenOp(const LLMEmbeddingTokenOpCargo& cargo)
    : BaseOp(OpType::kLLMEmbeddingToken), cargo_(cargo) {}

void LLMEmbeddingTokenOp::load(const std::shared_ptr<ParameterLoader>& ploader) {
  weight_ = Tensor((*ploader)[name() + ".weight"]);
}

void LLMEmbeddingTokenOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto shape = inputs[0].shape();  // [batch, seq]
  outputs.emplace_back(Tensor::empty({shape[0], shape[1], cargo_.hidden_size}, weight_.dtype(), inputs[0].device()));
}

LLMEmbeddingTokenOp::params_t LLMEmbeddingTokenOp::params() {
  params_t ret;
  ret.insert({name() + ".weight", weight_});
  return ret;
}

}  // namespace mllm
