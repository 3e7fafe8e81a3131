// Tensor, BaseOp::setup and the device-independent LinearOp.
#include <numeric>

#include "mllm/Core/AOps/LinearOp.hpp"
#include "mllm/Core/Tensor.hpp"
#include "mllm/Engine/Context.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "mllm/Utils/Log.hpp"

namespace mllm {

TensorStorage::~TensorStorage() {
  // kParams storage aliases a mapped file or caller memory and is never freed here
  // (reference: mllm/Core/TensorImpl.cpp:17-34).
  if (ptr_ && mem_type_ == kNormal) MllmEngineCtx::instance().mem()->free(this);
}

Tensor Tensor::empty(const shape_t& shape, DataTypes dtype, DeviceTypes device) {
  auto impl = std::make_shared<TensorViewImpl>();
  impl->shape_ = shape;
  impl->dtype_ = dtype;
  impl->storage_ = std::make_shared<TensorStorage>();
  impl->storage_->device_ = device;
  Tensor t(impl);
  impl->storage_->size_ = t.bytes();
  return t;
}

Tensor Tensor::wrap(void* ptr, const shape_t& shape, DataTypes dtype, DeviceTypes device,
                    std::shared_ptr<void> keep_alive) {
  Tensor t = empty(shape, dtype, device);
  t.impl_->storage_->ptr_ = ptr;
  t.impl_->storage_->mem_type_ = kParams;
  t.impl_->storage_->keep_alive_ = std::move(keep_alive);
  return t;
}

Tensor& Tensor::alloc() {
  if (!impl_->storage_->ptr_) MllmEngineCtx::instance().mem()->alloc(impl_->storage_);
  return *this;
}

size_t Tensor::numel() const {
  size_t n = 1;
  for (int32_t d : impl_->shape_) n *= static_cast<size_t>(d);
  return n;
}

void BaseOp::setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  (void)inputs;
  for (auto& o : outputs) o.alloc();
}

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
  MLLM_WARN("Can't parse Linear Impl Type: %s. Fallback to default impl.", type_str.c_str());
  return T::kDefault;
}

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

}  // namespace mllm
