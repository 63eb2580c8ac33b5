// sparse_conv2d operator: the 1x1 convolution over pruned weights in the
// NonZeroWeights / OcNonZeros / Diffs form.  Same inputs, outputs and
// attributes as the reference (lite/operators/sparse_conv_op.h:31-188).
#pragma once

#include <string>

#include "lite/core/op_lite.h"
#include "lite/core/profile/profiler.h"
#include "lite/operators/op_params.h"

namespace paddle {
namespace lite {
namespace operators {

class SparseConvOp : public OpLite {
 public:
  SparseConvOp() = default;
  explicit SparseConvOp(const std::string& type) : OpLite(type) {}

  bool CheckShape() const override;
  bool InferShapeImpl() const override;
  bool AttachImpl(const cpp::OpDesc& op_desc, lite::Scope* scope) override;
  void AttachKernel(KernelBase* kernel) override { kernel->SetParam(param_); }
  std::string DebugString() const override { return "sparse_conv2d"; }

  // Dense-counted multiply-accumulate operations, as the reference reports
  // them to its profiler (sparse_conv_op.h:41-63).
  float Macs() const;
  // What the op tells the profiler about one run: shapes, the
  // "1x1p<pad>s<stride>g<groups>d<dilation>[Bias]<Activation>" remark and the
  // dense-counted operations (sparse_conv_op.h:41-63; compiled there under
  // LITE_WITH_PROFILE only).
  void GetOpRuntimeInfo(paddle::lite::profile::OpCharacter* ch) const;
  const SparseConvParam& param() const { return param_; }

 private:
  mutable SparseConvParam param_;
};

}  // namespace operators
}  // namespace lite
}  // namespace paddle
