// calib: changes the precision of a tensor with a per-tensor scale; the op
// the quantisation passes place between an fp32 producer and an int8 consumer
// and back (reference: lite/operators/calib_op.{h,cc}).
#pragma once

#include <string>

#include "lite/core/op_lite.h"
#include "lite/operators/op_params.h"

namespace paddle {
namespace lite {
namespace operators {

class CalibOpLite : public OpLite {
 public:
  CalibOpLite() = default;
  explicit CalibOpLite(const std::string& type) : OpLite(type) {}
  bool CheckShape() const override {
    CHECK_OR_FALSE(param_.input);
    CHECK_OR_FALSE(param_.output);
    return true;
  }
  bool InferShapeImpl() const override {
    param_.output->Resize(param_.input->dims());
    param_.output->set_lod(param_.input->lod());
    return true;
  }
  bool AttachImpl(const cpp::OpDesc& d, Scope* scope) override;
  void AttachKernel(KernelBase* kernel) override { kernel->SetParam(param_); }
  std::string DebugString() const override { return "calib"; }

 private:
  mutable CalibParam param_;
};

}  // namespace operators
}  // namespace lite
}  // namespace paddle
