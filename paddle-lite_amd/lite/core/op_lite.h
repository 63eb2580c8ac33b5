// OpLite: operator base class; binds an OpDesc and a Scope to a parameter
// struct, infers output shapes, creates and feeds kernels
// (reference: lite/core/op_lite.h).
#pragma once

#include <list>
#include <memory>
#include <string>
#include <vector>

#include "lite/core/kernel.h"
#include "lite/core/op_desc.h"
#include "lite/core/scope.h"

namespace paddle {
namespace lite {

class OpLite {
 public:
  OpLite() = default;
  explicit OpLite(const std::string& type) : op_type_(type) {}
  virtual ~OpLite() = default;

  virtual bool CheckShape() const { return true; }
  virtual bool InferShapeImpl() const { return true; }
  virtual bool InferShape() { return InferShapeImpl(); }
  virtual bool AttachImpl(const cpp::OpDesc& desc, Scope* scope) = 0;
  virtual void AttachKernel(KernelBase* kernel) = 0;
  virtual std::string DebugString() const = 0;

  bool Attach(const cpp::OpDesc& desc, Scope* scope) {
    scope_ = scope;
    op_info_.reset(new OpInfo(desc));
    return AttachImpl(*op_info_, scope);
  }
  const OpInfo* op_info() const { return op_info_.get(); }
  const std::string& Type() const { return op_type_; }

  // Kernels registered for this op at the first valid place that has any.
  std::vector<std::unique_ptr<KernelBase>> CreateKernels(const std::vector<lite_api::Place>& places, const std::string& kernel_type = "");

 protected:
  Scope* scope_{nullptr};
  std::string op_type_;
  std::unique_ptr<OpInfo> op_info_;
};

}  // namespace lite
}  // namespace paddle
