// KernelBase / KernelLite: the interface every Lite kernel implements and the
// call order the runtime guarantees (reference: lite/core/kernel.h:43-200).
#pragma once

#include <any>
#include <memory>
#include <string>

#include "lite/api/paddle_place.h"
#include "lite/core/context.h"
#include "lite/utils/log.h"

namespace paddle {
namespace lite {

class KernelBase {
 public:
  virtual ~KernelBase() = default;

  // Once, after SetParam and SetContext.
  virtual void PrepareForRun() {}
  // Before every Run (e.g. when input shapes may have changed).
  virtual void ReInitWhenNeeded() {}
  virtual void Run() = 0;

  // reference: kernel.h:84-123
  void Launch() {
    if (is_first_epoch_) {
      PrepareForRun();
      is_first_epoch_ = false;
    }
    ReInitWhenNeeded();
    Run();
  }

  // The op hands the kernel a COPY of its parameter struct.
  template <typename T>
  void SetParam(T param) {
    param_ = param;
  }
  template <typename P>
  P& Param() const {
    P* p = std::any_cast<P>(&param_);
    CHECK(p != nullptr) << "kernel parameter has another type";
    return *p;
  }

  void SetContext(std::unique_ptr<KernelContext>&& ctx) { ctx_ = std::move(ctx); }
  KernelContext* mutable_context() { return ctx_.get(); }
  template <typename T>
  T* mutable_context_as() {
    return &ctx_->As<T>();
  }

  void set_op_type(const std::string& t) { op_type_ = t; }
  const std::string& op_type() const { return op_type_; }
  void set_alias(const std::string& a) { alias_ = a; }
  const std::string& alias() const { return alias_; }

  virtual lite_api::TargetType target() const = 0;
  virtual lite_api::PrecisionType precision() const = 0;
  virtual lite_api::DataLayoutType layout() const = 0;
  lite_api::Place place() const { return lite_api::Place(target(), precision(), layout()); }
  virtual std::string name() const = 0;
  // "op_type/alias", the key parameter types are registered under
  std::string key_with_alias() const { return op_type_ + "/" + alias_; }
  std::string summary() const { return op_type_ + ":" + lite_api::TargetToStr(target()) + "/" + lite_api::PrecisionToStr(precision()) + "/" + alias_; }

 protected:
  std::unique_ptr<KernelContext> ctx_;
  mutable std::any param_;
  std::string op_type_, alias_;
  bool is_first_epoch_{true};
};

template <lite_api::TargetType Target, lite_api::PrecisionType Precision, lite_api::DataLayoutType Layout = lite_api::DataLayoutType::kNCHW>
class KernelLite : public KernelBase {
 public:
  void Run() override { CHECK(false) << "Not Implemented"; }
  lite_api::TargetType target() const override { return Target; }
  lite_api::PrecisionType precision() const override { return Precision; }
  lite_api::DataLayoutType layout() const override { return Layout; }
  std::string name() const override { return op_type() + ":" + lite_api::TargetToStr(Target) + "/" + lite_api::PrecisionToStr(Precision); }
};

}  // namespace lite
}  // namespace paddle
