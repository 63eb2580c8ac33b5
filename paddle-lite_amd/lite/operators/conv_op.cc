#include "lite/operators/conv_op.h"

#include "lite/core/op_registry.h"

namespace paddle {
namespace lite {
namespace operators {

bool ConvOpLite::CheckShape() const {
  // lite/operators/conv_op.cc:25-41
  CHECK_OR_FALSE(param_.x);
  CHECK_OR_FALSE(param_.output);
  CHECK_OR_FALSE(param_.filter);
  const DDim& in = param_.x->dims();
  const DDim& f = param_.filter->dims();
  CHECK_OR_FALSE(in.size() == 4);
  CHECK_OR_FALSE(in.size() == f.size());
  CHECK_OR_FALSE(static_cast<size_t>(in.size()) - param_.strides.size() == 2U);
  CHECK_OR_FALSE(f.size() == 4);
  CHECK_OR_FALSE(in[1] == f[1] * param_.groups);
  CHECK_OR_FALSE(f[0] % param_.groups == 0);
  return true;
}

bool ConvOpLite::InferShapeImpl() const {
  // lite/operators/conv_op.cc:83-111 with explicit paddings (ConvOutputSize:
  // (in + pad0 + pad1 - (dilation * (k - 1) + 1)) / stride + 1)
  const DDim& in = param_.x->dims();
  const DDim& f = param_.filter->dims();
  std::vector<int64_t> out{in[0], f[0]};
  const auto& pads = *param_.paddings;
  const auto& dil = *param_.dilations;
  for (size_t i = 0; i < param_.strides.size(); ++i) {
    const int64_t dkernel = dil[i] * (f[i + 2] - 1) + 1;
    out.push_back((in[i + 2] + pads[2 * i] + pads[2 * i + 1] - dkernel) / param_.strides[i] + 1);
  }
  param_.output->Resize(DDim(out));
  param_.output->set_lod(param_.x->lod());
  return true;
}

bool ConvOpLite::AttachImpl(const cpp::OpDesc& d, Scope* scope) {
  // lite/operators/conv_op.h:60-200
  auto find = [&](const std::string& name) -> Tensor* {
    Variable* v = scope->FindVar(name);
    CHECK(v != nullptr) << "conv2d: variable " << name << " not found";
    return v->GetMutable<Tensor>();
  };
  param_ = ConvParam();
  param_.x = find(d.Input("Input").front());
  param_.filter = find(d.Input("Filter").front());
  param_.output = find(d.Output("Output").front());
  param_.strides = d.GetAttr<std::vector<int>>("strides");
  std::vector<int> pads = d.GetAttr<std::vector<int>>("paddings");
  param_.groups = d.GetAttr<int>("groups");
  param_.dilations = std::make_shared<std::vector<int>>(d.GetAttr<std::vector<int>>("dilations"));
  if (d.HasInput("Bias") && !d.Input("Bias").empty()) {
    if (Variable* v = scope->FindVar(d.Input("Bias").front())) param_.bias = v->GetMutable<Tensor>();
  }
  if (d.HasAttr("with_act") && d.GetAttr<bool>("with_act")) {
    ActivationParam& a = param_.activation_param;
    a.has_active = true;
    const std::string type = d.GetAttr<std::string>("act_type");
    using AT = lite_api::ActivationType;
    if (type == "relu") {
      a.active_type = AT::kRelu;
      param_.fuse_relu = true;
    } else if (type == "relu6") {
      a.active_type = AT::kRelu6;
      a.Relu_clipped_coef = d.GetAttr<float>("fuse_brelu_threshold");
    } else if (type == "leaky_relu") {
      a.active_type = AT::kLeakyRelu;
      a.Leaky_relu_alpha = d.GetAttr<float>("leaky_relu_alpha");
    } else if (type == "hard_swish") {
      a.active_type = AT::kHardSwish;
      a.hard_swish_threshold = d.GetAttr<float>("hard_swish_threshold");
      a.hard_swish_scale = d.GetAttr<float>("hard_swish_scale");
      a.hard_swish_offset = d.GetAttr<float>("hard_swish_offset");
    } else {
      LOG(FATAL) << "The fused conv only supports fuse with relu, leaky relu, hard_swish, while the given activation type is " << type;
    }
  }
  const OpInfo* info = dynamic_cast<const OpInfo*>(&d);
  if (info != nullptr && info->HasAttr("enable_int8")) {
    param_.enable_int8 = info->GetAttr<bool>("enable_int8");
    if (info->HasInputScale("Input0_scale", true)) param_.input_scale = info->GetInputScale("Input0_scale", true)[0];
    if (info->HasInputScale("Filter0_scale", true)) param_.weight_scale = info->GetInputScale("Filter0_scale", true);
    if (info->HasOutputScale("Output0_scale", true)) param_.output_scale = info->GetOutputScale("Output0_scale", true)[0];
  }
  if (pads.size() == 2) {
    pads = {pads[0], pads[0], pads[1], pads[1]};
  } else if (pads.size() != 4) {
    LOG(FATAL) << "Paddings size should be the same or twice as the input size.";
  }
  param_.paddings = std::make_shared<std::vector<int>>(pads);
  return true;
}

}  // namespace operators
}  // namespace lite
}  // namespace paddle

REGISTER_LITE_OP(depthwise_conv2d, paddle::lite::operators::ConvOpLite);
