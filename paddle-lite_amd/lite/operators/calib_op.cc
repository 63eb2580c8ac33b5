#include "lite/operators/calib_op.h"

#include "lite/core/op_registry.h"

namespace paddle {
namespace lite {
namespace operators {

// reference: CalibOpLite::AttachImpl (lite/operators/calib_op.cc:52-66):
// Input / Out by name, optional float attribute "scale".
bool CalibOpLite::AttachImpl(const cpp::OpDesc& d, Scope* scope) {
  Variable* x = scope->FindVar(d.Input("Input").front());
  Variable* out = scope->FindVar(d.Output("Out").front());
  CHECK(x != nullptr) << "Input(X) of CalibOp should not be null.";
  CHECK(out != nullptr) << "Output(Out) of CalibOp should not be null.";
  param_.input = x->GetMutable<Tensor>();
  param_.output = out->GetMutable<Tensor>();
  if (d.HasAttr("scale")) param_.scale = d.GetAttr<float>("scale");
  return true;
}

}  // namespace operators
}  // namespace lite
}  // namespace paddle

REGISTER_LITE_OP(calib, paddle::lite::operators::CalibOpLite);
