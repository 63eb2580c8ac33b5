#include "lite/operators/io_copy_op.h"

#include "lite/core/op_registry.h"

namespace paddle {
namespace lite {
namespace operators {

bool IoCopyOp::AttachImpl(const cpp::OpDesc& d, Scope* scope) {
  Variable* x = scope->FindVar(d.Input("Input").front());
  CHECK(x != nullptr) << "io_copy input not found";
  param_.x = x->GetMutable<Tensor>();
  param_.y = scope->Var(d.Output("Out").front())->GetMutable<Tensor>();
  if (d.HasAttr("process_type")) param_.process_type = d.GetAttr<int>("process_type");
  return true;
}

}  // namespace operators
}  // namespace lite
}  // namespace paddle

REGISTER_LITE_OP(io_copy, paddle::lite::operators::IoCopyOp);
