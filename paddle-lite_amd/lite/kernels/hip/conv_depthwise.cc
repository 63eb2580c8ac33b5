// int8 depthwise 3x3 convolution kernels of TARGET(kHIP), the counterpart of
// DepthwiseConv<PRECISION(kInt8), PRECISION(kFloat | kInt8)>
// (lite/kernels/arm/conv_depthwise.cc:158-200, :257-322 PrepareForRun,
// :359-412 Run) as ConvCompute picks it for groups == channels
// (lite/kernels/arm/conv_compute.cc), registered like the reference's
// depthwise_conv2d int8 kernels (aliases int8_out / fp32_out,
// conv_compute.cc:252-300).
#include "lite/core/op_registry.h"
#include "lite/kernels/hip/pair_launch.h"
#include "lite/operators/op_params.h"
#include "pl_sparse_conv.h"

namespace paddle {
namespace lite {
namespace kernels {
namespace hip {

template <PrecisionType O>
class DepthwiseConvInt8 : public KernelLite<TARGET(kHIP), PRECISION(kInt8)>, public PairLaunch {
 public:
  using param_t = operators::ConvParam;
  ~DepthwiseConvInt8() override {
    if (handle_) pl_dwconv3x3_destroy(handle_);
  }

  void PrepareForRun() override {
    auto& param = this->template Param<param_t>();
    const DDim& w = param.filter->dims();
    const int oc = static_cast<int>(w[0]);
    CHECK(w[2] == 3 && w[3] == 3) << "this type dw conv not impl";
    CHECK(param.groups == oc && w[1] == 1) << "depthwise: groups must equal the channel count";
    const auto& pads = *param.paddings;
    CHECK(pads[0] == pads[1] && pads[0] == pads[2] && pads[0] == pads[3] && (pads[0] == 0 || pads[0] == 1)) << "depthwise 3x3: padding 0 or 1 on all sides";
    CHECK(param.strides[0] == param.strides[1] && (param.strides[0] == 1 || param.strides[0] == 2)) << "depthwise 3x3: stride 1 or 2";
    CHECK((*param.dilations)[0] == 1 && (*param.dilations)[1] == 1) << "depthwise 3x3: dilation 1";
    constexpr bool kInt8Out = O == PRECISION(kInt8);
    const float in_scale = param.input_scale, out_scale = param.output_scale;
    const auto& scale = param.weight_scale;
    CHECK(scale.size() == 1 || static_cast<int>(scale.size()) == oc) << "weights scale size must = filter size or = 1";
    w_scale_.resize(oc);
    for (int i = 0; i < oc; ++i) {
      const float ws = scale.size() == 1 ? scale[0] : scale[i];
      w_scale_[i] = kInt8Out ? ws * in_scale / out_scale : ws * in_scale;
    }
    const float* bias = param.bias ? param.bias->template data<float>() : nullptr;
    if (kInt8Out && param.bias) {
      bias_.resize(oc);
      for (int i = 0; i < oc; ++i) bias_[i] = bias[i] / out_scale;
      bias = bias_.data();
    }
    // the parameter is this kernel's own copy, changed in place like the reference does
    operators::ActivationParam& act = param.activation_param;
    if (kInt8Out && act.active_type == lite_api::ActivationType::kRelu6) act.Relu_clipped_coef = act.Relu_clipped_coef / out_scale;
    if (kInt8Out && act.active_type == lite_api::ActivationType::kHardSwish) {
      act.hard_swish_offset = act.hard_swish_offset / out_scale;
      act.hard_swish_threshold = act.hard_swish_threshold / out_scale;
    }
    pl_dwconv_desc d{};
    d.struct_size = sizeof(d);
    d.kind = kInt8Out ? PL_KIND_INT8_INT8 : PL_KIND_INT8_FP32;
    d.channels = oc;
    d.stride = param.strides[0];
    d.pad = pads[0];
    d.weights = param.filter->template data<int8_t>();
    d.scale = w_scale_.data();
    d.bias = bias;
    d.act.type = act.has_active ? static_cast<int32_t>(act.active_type) : PL_ACT_NONE;
    d.act.relu6_coef = act.Relu_clipped_coef;
    d.act.leaky_alpha = act.Leaky_relu_alpha;
    d.act.hs_scale = act.hard_swish_scale;
    d.act.hs_offset = act.hard_swish_offset;
    d.act.hs_threshold = act.hard_swish_threshold;
    if (handle_) pl_dwconv3x3_destroy(handle_);
    handle_ = nullptr;
    const int rc = pl_dwconv3x3_prepare(&d, &handle_);
    if (rc != PL_OK) LOG(FATAL) << "pl_dwconv3x3_prepare failed (" << rc << "): " << pl_last_error();
  }

  void Run() override {
    auto& param = this->template Param<param_t>();
    CHECK(param.x->target() == TargetType::kHIP) << "depthwise_conv2d: Input is not on the device";
    const DDim& xd = param.x->dims();
    void* out = O == PRECISION(kInt8) ? static_cast<void*>(param.output->template mutable_data<int8_t>(TargetType::kHIP)) : static_cast<void*>(param.output->template mutable_data<float>(TargetType::kHIP));
    const int rc = pl_dwconv3x3_run(handle_, static_cast<const int8_t*>(param.x->raw_data()), out, static_cast<int32_t>(xd[0]), static_cast<int32_t>(xd[2]), static_cast<int32_t>(xd[3]),
                                    this->ctx_->template As<HIPContext>().stream());
    if (rc != PL_OK) LOG(FATAL) << "pl_dwconv3x3_run failed (" << rc << "): " << pl_last_error();
  }

  // Second end of a pair launch (pair_launch.h): only the int8 -> int8 kernel can be one.
  PairLaunch::Role pair_role() const override { return PairLaunch::kSecond; }
  bool pair_endpoint(PairEndpoint* e) override {
    if (handle_ == nullptr || O != PRECISION(kInt8)) return false;
    auto& param = this->template Param<param_t>();
    if (param.x->target() != TargetType::kHIP) return false;
    const DDim& xd = param.x->dims();
    if (xd.size() != 4) return false;
    e->handle = handle_;
    e->x = param.x->raw_data();
    e->out = param.output->template mutable_data<int8_t>(TargetType::kHIP);
    e->batch = static_cast<int>(xd[0]);
    e->h = static_cast<int>(xd[2]);
    e->w = static_cast<int>(xd[3]);
    e->stream = this->ctx_->template As<HIPContext>().stream();
    return true;
  }

 private:
  pl_dwconv_handle* handle_ = nullptr;
  std::vector<float> w_scale_, bias_;
};

}  // namespace hip
}  // namespace kernels
}  // namespace lite
}  // namespace paddle

typedef paddle::lite::kernels::hip::DepthwiseConvInt8<PRECISION(kInt8)> DepthwiseConvInt8_Int8;
typedef paddle::lite::kernels::hip::DepthwiseConvInt8<PRECISION(kFloat)> DepthwiseConvInt8_Fp32;

REGISTER_LITE_KERNEL(depthwise_conv2d, kHIP, kInt8, kNCHW, DepthwiseConvInt8_Int8, int8_out)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kInt8))})
    .BindInput("Bias", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kFloat))})
    .BindInput("Filter", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt8))})
    .BindOutput("Output", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kInt8))})
    .Finalize();

REGISTER_LITE_KERNEL(depthwise_conv2d, kHIP, kInt8, kNCHW, DepthwiseConvInt8_Fp32, fp32_out)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kInt8))})
    .BindInput("Bias", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kFloat))})
    .BindInput("Filter", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt8))})
    .BindOutput("Output", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kFloat))})
    .Finalize();
