// depthwise_conv2d operator, as much of the reference's ConvOpLite
// (lite/operators/conv_op.{h,cc}, registered for conv2d, conv3d and
// depthwise_conv2d) as the int8 depthwise 3x3 kernels of TARGET(kHIP) need:
// Input / Filter / Bias / Output, strides, paddings, dilations, groups, the
// fused activation and the int8 scales.
#pragma once

#include <string>

#include "lite/core/op_lite.h"
#include "lite/operators/op_params.h"

namespace paddle {
namespace lite {
namespace operators {

class ConvOpLite : public OpLite {
 public:
  ConvOpLite() = default;
  explicit ConvOpLite(const std::string& type) : OpLite(type) {}

  bool CheckShape() const override;
  bool InferShapeImpl() const override;
  bool AttachImpl(const cpp::OpDesc& op_desc, lite::Scope* scope) override;
  void AttachKernel(KernelBase* kernel) override { kernel->SetParam(param_); }
  std::string DebugString() const override { return "conv2d"; }
  const ConvParam& param() const { return param_; }

 private:
  mutable ConvParam param_;
};

}  // namespace operators
}  // namespace lite
}  // namespace paddle
