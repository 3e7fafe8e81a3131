// Linear: cargo, implementation selector and the device-independent part of the op
// (reference: mllm/Core/AOps/LinearOp.hpp:17-99, mllm/Core/AOps/LinearOp.cpp:17-106).
#pragma once

#include <string>

#include "mllm/Core/AOps/BaseOp.hpp"

namespace mllm {

// Same enumerators and values as the reference (LinearOp.hpp:17-35): model configs and quantizer
// configs name an implementation by string, the op switches on the value. 3..8 are the six tile
// variants of the W4A32 family KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk - on this backend they all
// run the same kernels (a tile only selected an Arm micro-kernel and its packed layout).
enum class LinearOpImplType {
  kDefault = 0,
  kKai_Start = 1,
  kKaiLinear_fp16_fp16_fp16p_mxk_kxn = 2,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x8_qsi4c32p4x8_1x4x32 = 3,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x8_qsi4c32p8x8_1x8x32 = 4,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p4x8_8x4x32 = 5,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p4x8_16x4x32 = 6,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p8x8_4x8x32 = 7,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x4_qsi4c32p4x4_1x4 = 8,
  KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p1x8_qai4c32p4x8_1x4 = 9,
  KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p4x4_qai4c32p4x4_8x4 = 10,
  KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p4x8_qai4c32p4x8_8x4_i8mm = 11,
  kKai_End = 256,
};

inline bool isW4A32ImplType(LinearOpImplType t) {
  const int v = static_cast<int>(t);
  return v >= 3 && v <= 8;
}

struct LinearOpCargo : public BaseOpCargo<LinearOpCargo> {
  int32_t in_channels = 0;
  int32_t out_channels = 0;
  bool bias = true;
  bool transpose = false;
  LinearOpImplType impl_type_ = LinearOpImplType::kDefault;

  // "<family>:<tile>" -> enum; unknown strings warn and fall back to kDefault (LinearOp.cpp:53-55).
  static LinearOpImplType parseLinearOpImplTypeStr(const std::string& type_str);
};

class LinearOp : public BaseOp {
 public:
  explicit LinearOp(const LinearOpCargo& cargo) : BaseOp(OpType::kLinear), cargo_(cargo) {}

  // weight = "<name>.weight", bias = "<name>.bias" when cargo.bias (LinearOp.cpp:60-63)
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;
  // output = input shape with the last dimension replaced by out_channels (LinearOp.cpp:84-94)
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  params_t params() override;

  Tensor& weight() { return weight_; }
  Tensor& bias() { return bias_; }
  [[nodiscard]] const LinearOpCargo& cargo() const { return cargo_; }

 protected:
  Tensor weight_;
  Tensor bias_;
  LinearOpCargo cargo_;
};

}  // namespace mllm
