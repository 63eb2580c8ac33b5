// io_copy: moves a tensor between host and device memory; the op
// type_target_cast_pass inserts where a kernel's declared argument target
// differs from where the tensor lives (reference: lite/operators/io_copy_op.{h,cc}).
#pragma once

#include <string>

#include "lite/core/op_lite.h"
#include "lite/operators/op_params.h"

namespace paddle {
namespace lite {
namespace operators {

class IoCopyOp : public OpLite {
 public:
  IoCopyOp() = default;
  explicit IoCopyOp(const std::string& type) : OpLite(type) {}
  bool CheckShape() const override {
    CHECK_OR_FALSE(param_.x);
    CHECK_OR_FALSE(param_.y);
    return true;
  }
  bool InferShapeImpl() const override {
    param_.y->Resize(param_.x->dims());
    param_.y->set_lod(param_.x->lod());
    return true;
  }
  bool AttachImpl(const cpp::OpDesc& d, Scope* scope) override;
  void AttachKernel(KernelBase* kernel) override { kernel->SetParam(param_); }
  std::string DebugString() const override { return "io_copy"; }

 private:
  mutable IoCopyParam param_;
};

}  // namespace operators
}  // namespace lite
}  // namespace paddle
