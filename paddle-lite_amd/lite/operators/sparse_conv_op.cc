#include "lite/operators/sparse_conv_op.h"

#include <algorithm>

#include "lite/core/op_registry.h"

namespace paddle {
namespace lite {
namespace operators {

namespace {

Tensor* MustFind(Scope* scope, const cpp::OpDesc& d, const std::string& arg, bool input) {
  const auto names = input ? d.Input(arg) : d.Output(arg);
  CHECK(!names.empty()) << "sparse_conv2d: argument " << arg << " is empty";
  Variable* v = scope->FindVar(names.front());
  CHECK(v != nullptr) << "sparse_conv2d: variable " << names.front() << " not found";
  return v->GetMutable<Tensor>();
}

// Reads the fused-activation attributes written by the conv+activation fusion
// (reference: sparse_conv_op.h:99-143).
void ReadActivation(const cpp::OpDesc& d, Scope* scope, SparseConvParam* p) {
  if (!(d.HasAttr("with_act") && d.GetAttr<bool>("with_act"))) return;
  ActivationParam& a = p->activation_param;
  a.has_active = true;
  const std::string type = d.GetAttr<std::string>("act_type");
  using AT = lite_api::ActivationType;
  if (type == "relu") {
    a.active_type = AT::kRelu;
    p->fuse_relu = true;
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
  } else if (type == "hard_sigmoid") {
    // accepted by the op although no sparse kernel implements it
    a.active_type = AT::kHardSigmoid;
    a.hard_sigmoid_slope = d.GetAttr<float>("slope");
    a.hard_sigmoid_offset = d.GetAttr<float>("offset");
  } else if (type == "prelu") {
    a.active_type = AT::kPRelu;
    a.Prelu_mode = d.GetAttr<std::string>("prelu_mode");
    Variable* v = scope->FindVar(d.Input("Prelu_alpha").front());
    CHECK(v != nullptr) << "Prelu_alpha variable not found";
    a.Prelu_alpha = v->GetMutable<Tensor>();
  } else {
    LOG(FATAL) << "The fused conv only supports fuse with relu, leaky relu, relu6, while the given activation type is " << type;
  }
}

}  // namespace

bool SparseConvOp::CheckShape() const {
  CHECK_OR_FALSE(param_.x);
  CHECK_OR_FALSE(param_.output);
  CHECK_OR_FALSE(param_.nonzero_weights);
  CHECK_OR_FALSE(param_.oc_nonzeros);
  CHECK_OR_FALSE(param_.diffs);
  return true;
}

bool SparseConvOp::InferShapeImpl() const {
  const DDim& in = param_.x->dims();
  // The pass sizes OcNonZeros to the output channel count in both layouts
  // (reference: sparse_conv_op.cc:46-65).
  std::vector<int64_t> out{in[0], param_.oc_nonzeros->dims()[0]};
  const auto& pads = *param_.paddings;
  const auto& dil = *param_.dilations;
  for (size_t i = 0; i < param_.strides.size(); ++i) {
    const int dkernel = dil[i] * (1 - 1) + 1;  // filter size is 1
    out.push_back((in[i + 2] + pads[2 * i] + pads[2 * i + 1] - dkernel) / param_.strides[i] + 1);
  }
  param_.output->Resize(DDim(out));
  param_.output->set_lod(param_.x->lod());
  return true;
}

bool SparseConvOp::AttachImpl(const cpp::OpDesc& d, Scope* scope) {
  param_ = SparseConvParam();
  param_.x = MustFind(scope, d, "Input", true);
  param_.nonzero_weights = MustFind(scope, d, "NonZeroWeights", true);
  param_.oc_nonzeros = MustFind(scope, d, "OcNonZeros", true);
  param_.diffs = MustFind(scope, d, "Diffs", true);
  param_.output = MustFind(scope, d, "Output", false);

  param_.strides = d.GetAttr<std::vector<int>>("strides");
  std::vector<int> pads = d.GetAttr<std::vector<int>>("paddings");
  param_.groups = d.GetAttr<int>("groups");
  param_.dilations = std::make_shared<std::vector<int>>(d.GetAttr<std::vector<int>>("dilations"));

  if (d.HasInput("Bias")) {
    const auto names = d.Input("Bias");
    if (!names.empty()) {
      if (Variable* v = scope->FindVar(names.front())) param_.bias = v->GetMutable<Tensor>();
    }
  }
  ReadActivation(d, scope, &param_);
  if (d.HasAttr("first_ic")) param_.first_ic = d.GetAttr<int>("first_ic");
  if (d.HasAttr("flag_semi")) param_.flag_semi = d.GetAttr<int>("flag_semi");

  // int8: scales travel as "<Arg>0_scale" attributes (sparse_conv_op.h:151-166)
  const OpInfo* info = dynamic_cast<const OpInfo*>(&d);
  if (info != nullptr && info->HasAttr("enable_int8")) {
    param_.enable_int8 = info->GetAttr<bool>("enable_int8");
    if (info->HasInputScale("Input0_scale", true)) param_.input_scale = info->GetInputScale("Input0_scale", true)[0];
    if (info->HasInputScale("Filter0_scale", true)) param_.weight_scale = info->GetInputScale("Filter0_scale", true);
    if (info->HasOutputScale("Output0_scale", true)) param_.output_scale = info->GetOutputScale("Output0_scale", true)[0];
  }

  // {pad_h, pad_w} -> {top, bottom, left, right}
  if (pads.size() == 2) {
    pads = {pads[0], pads[0], pads[1], pads[1]};
  } else if (pads.size() != 4) {
    LOG(FATAL) << "Paddings size should be the same or twice as the input size.";
  }
  param_.paddings = std::make_shared<std::vector<int>>(pads);
  return true;
}

void SparseConvOp::GetOpRuntimeInfo(paddle::lite::profile::OpCharacter* ch) const {
  // names as lite_api::ActivationTypeToStr prints them (lite/api/paddle_place.cc:48-69), including
  // the table's shift against the enum from position 6 on (hard_swish = 10 prints as "Abs")
  static const char* const kActNames[] = {"unk", "Relu", "Relu6", "PRelu", "LeakyRelu", "Sigmoid", "Silu", "Tanh", "Swish", "Exp", "Abs", "HardSwish", "Reciprocal", "ThresholdedRelu", "Elu", "HardSigmoid", "log"};
  const DDim& filter_dims = param_.oc_nonzeros->dims();
  const DDim& input_dims = param_.x->dims();
  const DDim& output_dims = param_.output->dims();
  ch->op_type = "sparse_conv2d";
  ch->input_shape = ch->DimToStr(input_dims);
  ch->output_shape = ch->DimToStr(output_dims);
  ch->filter_shape = ch->DimToStr(filter_dims) + "x" + std::to_string(input_dims[1]) + "x1x1";
  const int act = static_cast<int>(param_.activation_param.active_type);
  CHECK(act >= 0 && act < static_cast<int>(sizeof(kActNames) / sizeof(kActNames[0]))) << "unknown activation type " << act;
  ch->remark = std::string("1x1p") + std::to_string((*param_.paddings)[0]) + "s" + std::to_string(param_.strides[0]) + "g" + std::to_string(param_.groups) + "d" + std::to_string((*param_.dilations)[0]) +
               (param_.bias ? "Bias" : "") + kActNames[act];
  ch->macs = Macs();
}

float SparseConvOp::Macs() const {
  return 2.f * param_.output->dims().production() * param_.x->dims()[1] / param_.groups;
}

}  // namespace operators
}  // namespace lite
}  // namespace paddle

REGISTER_LITE_OP(sparse_conv2d, paddle::lite::operators::SparseConvOp);
