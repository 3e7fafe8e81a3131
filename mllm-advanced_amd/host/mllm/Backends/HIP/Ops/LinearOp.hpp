// W4A32 Linear on MI355X behind the engine's LinearOp interface
// (reference counterpart: mllm/Backends/Arm/Ops/LinearOp.hpp:15-29, LinearOp.cpp:22-134,235-265).
#pragma once

#include "mllm/Core/AOps/D2HOp.hpp"
#include "mllm/Core/AOps/LinearOp.hpp"

namespace mllm::hip {

class HipLinearOp final : public LinearOp {
 public:
  explicit HipLinearOp(const LinearOpCargo& cargo);

  // Uploads the layer's weight and turns it into the device blob. Accepted "<name>.weight":
  //   * kFp32 [out, in]: quantised on the device exactly as the reference's offline quantizer
  //     does (bias = "<name>.bias", kFp32 [out], when cargo.bias);
  //   * kInt8 [bytes] in this build's row-major W4 format: out*in/2 nibble bytes, out*in/32 bf16
  //     scales, out f32 bias values (what quantizeLinearForFile() emits; the bias tensor in the
  //     file is then a 1-byte placeholder, as in the reference's quantised files).
  //   * int8 [ceil(out/nr)*nr * (in/32 * 18 + 8)]: the blob the reference's Arm quantizer writes for
  //     the op's tile (KleidiAI's packed layout, nr rows interleaved); it is un-interleaved on the
  //     device and repacked. That layout is restated from KleidiAI's published packing loop, which
  //     the reference tree does not contain: parity unpinned.
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;

  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;

  // Size in bytes of the row-major W4 file format for an [N][K] layer.
  static size_t nativeBlobBytes(int N, int K);

 private:
  Tensor workspace_;  // grown on demand, kept between calls
};

class HipLinearOpFactory : public TypedOpFactory<OpType::kLinear, LinearOpCargo> {
 public:
  std::shared_ptr<BaseOp> createOpImpl(const LinearOpCargo& cargo) override {
    return std::make_shared<HipLinearOp>(cargo);
  }
};

// Device -> host copy as an op (reference: mllm/Core/AOps/D2HOp.hpp, mllm/Backends/CUDA/Ops/D2HOp.cpp:18-22);
// Tensor::cpu() dispatches it with from_device_type = the tensor's device, to_device_type = kCPU.
class HipD2HOp final : public D2HOp {
 public:
  explicit HipD2HOp(const D2HOpCargo& cargo);
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

class HipD2HOpFactory : public TypedOpFactory<OpType::kD2H, D2HOpCargo> {
 public:
  std::shared_ptr<BaseOp> createOpImpl(const D2HOpCargo& cargo) override {
    return std::make_shared<HipD2HOp>(cargo);
  }
};

// Offline step of the quantizer tool for one layer: f32 weight [N][K] (+ optional f32 bias [N])
// on the host -> host tensor holding the row-major W4 file format. Runs the quantizer kernel on
// the device (bit-exact with the reference's scalar quantizer). Counterpart of
// KQP_linear_f32_qai8dxp_qsi4c32p_mxk_nxk::quantize (mllm/Backends/Arm/Passes/KaiQuantizationPass.cpp:104-187).
Tensor quantizeLinearForFile(const Tensor& weight_f32, const Tensor& bias_f32_or_nil);

}  // namespace mllm::hip
