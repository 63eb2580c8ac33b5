#include "lite/kernels/hip/sparse_conv_compute.h"

#include "pl_sparse_conv.h"
#include "lite/core/op_registry.h"

namespace paddle {
namespace lite {
namespace kernels {
namespace hip {

namespace {
bool g_reference_quirks = true;

pl_activation ToAbi(const operators::ActivationParam& a) {
  pl_activation p;
  p.type = a.has_active ? static_cast<int32_t>(a.active_type) : PL_ACT_NONE;
  p.relu6_coef = a.Relu_clipped_coef;
  p.leaky_alpha = a.Leaky_relu_alpha;
  p.hs_scale = a.hard_swish_scale;
  p.hs_offset = a.hard_swish_offset;
  p.hs_threshold = a.hard_swish_threshold;
  return p;
}

// weight_scale broadcast to one value per output channel
// (lite/kernels/arm/sparse_conv_compute.cc:36-46)
std::vector<float> PerChannelScales(const operators::SparseConvParam& param) {
  std::vector<float> s = param.weight_scale;
  const size_t oc = static_cast<size_t>(param.oc_nonzeros->dims()[0]);
  if (s.size() != 1 && s.size() != oc) {
    LOG(FATAL) << "weights scale size " << s.size() << " must equal to filter size " << oc;
  }
  if (s.size() == 1) s.resize(oc, s[0]);
  return s;
}

// The device kernels compute a 1x1 / stride 1 / pad 0 / dilation 1 / group 1
// convolution and size their reads from the output's H*W.  The detect pass
// only creates the op under these conditions
// (lite/core/optimizer/mir/sparse_conv_detect_pass.cc:596-640), but an op
// description loaded from a model file can say anything, and the op's own
// InferShape honours strides and paddings: refuse what would make the kernel
// read outside the input.
void CheckGeometry(const operators::SparseConvParam& param) {
  for (int s : param.strides) CHECK_EQ(s, 1) << "sparse_conv2d(kHIP): strides must be 1";
  CHECK(param.paddings != nullptr && param.dilations != nullptr) << "sparse_conv2d(kHIP): paddings / dilations unset";
  for (int p : *param.paddings) CHECK_EQ(p, 0) << "sparse_conv2d(kHIP): paddings must be 0";
  for (int d : *param.dilations) CHECK_EQ(d, 1) << "sparse_conv2d(kHIP): dilations must be 1";
  CHECK_EQ(param.groups, 1) << "sparse_conv2d(kHIP): groups must be 1";
  CHECK_EQ(param.x->dims().size(), 4u) << "sparse_conv2d(kHIP): Input must be NCHW";
}
}  // namespace

void SetSparseConvReferenceQuirks(bool on) { g_reference_quirks = on; }
bool SparseConvReferenceQuirks() { return g_reference_quirks; }

template <PrecisionType P, PrecisionType O>
SparseConvCompute<P, O>::~SparseConvCompute() {
  if (handle_) pl_sparse_conv_destroy(handle_);
}

template <PrecisionType P, PrecisionType O>
void SparseConvCompute<P, O>::Upload(int kind) {
  auto& param = this->template Param<param_t>();
  CHECK(param.x && param.nonzero_weights && param.oc_nonzeros && param.diffs) << "sparse_conv2d: unset input";
  CheckGeometry(param);
  const DDim& xd = param.x->dims();
  ic_ = xd[1];
  pl_sparse_conv_desc d{};
  d.struct_size = sizeof(d);
  d.kind = kind;
  d.flag_semi = param.flag_semi;
  d.first_ic = param.first_ic;
  d.oc = static_cast<int32_t>(param.oc_nonzeros->dims()[0]);
  d.ic = static_cast<int32_t>(xd[1]);
  d.im_size = static_cast<int32_t>(xd[2] * xd[3]);
  d.algo = PL_ALGO_AUTO;
  d.nonzero_weights = param.nonzero_weights->raw_data();
  d.n_weights = param.nonzero_weights->numel();
  d.oc_nonzeros = param.oc_nonzeros->template data<uint32_t>();
  d.diffs = param.diffs->template data<int32_t>();
  d.n_diffs = param.diffs->numel();
  d.scale = w_scale_.empty() ? nullptr : w_scale_.data();
  const Tensor* bias = flag_trans_bias_ ? &bias_ : param.bias;
  d.bias = bias ? bias->template data<float>() : nullptr;
  d.act = ToAbi(param.activation_param);
  if (kind == PL_KIND_INT8_INT8 && g_reference_quirks && d.act.type == PL_ACT_HARD_SWISH) {
    // second division, done inside the reference's math function
    d.act.hs_offset = d.act.hs_offset / param.output_scale;
    d.act.hs_threshold = d.act.hs_threshold / param.output_scale;
  }
  if (handle_) {
    pl_sparse_conv_destroy(handle_);
    handle_ = nullptr;
  }
  const int rc = pl_sparse_conv_prepare(&d, &handle_);
  if (rc != PL_OK) LOG(FATAL) << "pl_sparse_conv_prepare failed (" << rc << "): " << pl_last_error();
}

template <>
void SparseConvCompute<PRECISION(kFloat), PRECISION(kFloat)>::PrepareForRun() {
  Upload(PL_KIND_FP32);
}

template <>
void SparseConvCompute<PRECISION(kInt8), PRECISION(kFloat)>::PrepareForRun() {
  auto& param = this->Param<param_t>();
  w_scale_ = PerChannelScales(param);
  for (float& s : w_scale_) s *= param.input_scale;
  Upload(PL_KIND_INT8_FP32);
}

template <>
void SparseConvCompute<PRECISION(kInt8), PRECISION(kInt8)>::PrepareForRun() {
  auto& param = this->Param<param_t>();
  w_scale_ = PerChannelScales(param);
  const float in_scale = param.input_scale, out_scale = param.output_scale;
  for (float& s : w_scale_) s = s * in_scale / out_scale;
  if (param.bias) {
    bias_.Resize(param.bias->dims());
    float* dst = bias_.mutable_data<float>(TargetType::kHost);
    const float* src = param.bias->data<float>();
    for (int64_t i = 0; i < bias_.numel(); ++i) dst[i] = src[i] / out_scale;
    flag_trans_bias_ = true;
  }
  // the activation constants move to the output's quantised domain, in the
  // kernel's own copy of the parameters
  auto& act = param.activation_param;
  using AT = lite_api::ActivationType;
  if (act.active_type == AT::kRelu6) act.Relu_clipped_coef /= out_scale;
  if (act.active_type == AT::kLeakyRelu && g_reference_quirks) act.Leaky_relu_alpha /= out_scale;
  if (act.active_type == AT::kHardSwish) {
    act.hard_swish_scale /= out_scale;
    act.hard_swish_offset /= out_scale;
    act.hard_swish_threshold /= out_scale;
  }
  Upload(PL_KIND_INT8_INT8);
}

// Half precision: the reference converts the fp32 weights and bias in place
// and halves the byte offsets
// (lite/kernels/arm/sparse_conv_compute.cc:270-304); here the library does
// the conversion when it builds its device-side form, the host tensors stay
// as the pass wrote them.
template <>
void SparseConvCompute<PRECISION(kFP16), PRECISION(kFP16)>::PrepareForRun() {
  Upload(PL_KIND_FP16);
}

template <PrecisionType P, PrecisionType O>
void SparseConvCompute<P, O>::Run() {
  auto& param = this->template Param<param_t>();
  auto& ctx = this->ctx_->template As<HIPContext>();
  CHECK(handle_ != nullptr) << "PrepareForRun was not called";
  CHECK(param.x->target() == TargetType::kHIP) << "sparse_conv2d(kHIP): Input must live on the device (io_copy missing?)";
  CheckGeometry(param);
  const DDim& xd = param.x->dims();
  const DDim& od = param.output->dims();
  CHECK_EQ(od.size(), 4u) << "sparse_conv2d(kHIP): Output must be NCHW";
  CHECK_EQ(xd[1], ic_) << "sparse_conv2d(kHIP): Input has " << xd[1] << " channels, the weights were prepared for " << ic_;
  CHECK(xd[0] == od[0] && xd[2] * xd[3] == od[2] * od[3]) << "sparse_conv2d(kHIP): Input and Output differ in batch or H*W";
  const int batch = static_cast<int>(xd[0]);
  const int im_size = static_cast<int>(od[2] * od[3]);
  void* out = (O == PRECISION(kFloat)) ? static_cast<void*>(param.output->template mutable_data<float>(TargetType::kHIP))
              : (O == PRECISION(kFP16)) ? static_cast<void*>(param.output->template mutable_data<uint16_t>(TargetType::kHIP))
                                        : static_cast<void*>(param.output->template mutable_data<int8_t>(TargetType::kHIP));
  const int rc = pl_sparse_conv_run(handle_, param.x->raw_data(), out, batch, im_size, ctx.stream());
  if (rc != PL_OK) LOG(FATAL) << "pl_sparse_conv_run failed (" << rc << "): " << pl_last_error();
  last_batch_ = batch;
  last_im_size_ = im_size;
}

template <PrecisionType P, PrecisionType O>
bool SparseConvCompute<P, O>::pair_endpoint(PairEndpoint* e) {
  if (handle_ == nullptr || P != PRECISION(kInt8) || O != PRECISION(kInt8)) return false;
  auto& param = this->template Param<param_t>();
  if (param.x->target() != TargetType::kHIP) return false;
  CheckGeometry(param);
  const DDim& xd = param.x->dims();
  if (xd.size() != 4 || xd[1] != ic_) return false;
  e->handle = handle_;
  e->x = param.x->raw_data();
  e->out = param.output->template mutable_data<int8_t>(TargetType::kHIP);
  e->batch = static_cast<int>(xd[0]);
  e->h = static_cast<int>(xd[2]);
  e->w = static_cast<int>(xd[3]);
  e->stream = this->ctx_->template As<HIPContext>().stream();
  return true;
}

template <PrecisionType P, PrecisionType O>
std::string SparseConvCompute<P, O>::kernel_func_name() const {
  if (handle_ == nullptr || last_batch_ < 0) return "NotImplForSparseConv";
  static const char* const kAlgo[] = {"auto", "row_walk", "block_mfma", "image_mfma"};
  const int algo = pl_sparse_conv_algo_for(handle_, last_batch_, last_im_size_);
  return std::string("pl_sparse_conv_run/") + (algo >= 0 && algo <= 3 ? kAlgo[algo] : "unknown");
}

template class SparseConvCompute<PRECISION(kFloat), PRECISION(kFloat)>;
template class SparseConvCompute<PRECISION(kInt8), PRECISION(kFloat)>;
template class SparseConvCompute<PRECISION(kInt8), PRECISION(kInt8)>;
template class SparseConvCompute<PRECISION(kFP16), PRECISION(kFP16)>;

}  // namespace hip
}  // namespace kernels
}  // namespace lite
}  // namespace paddle

// Same op type, argument names and aliases as the ARM registrations
// (lite/kernels/arm/sparse_conv_compute.cc:369-430).  Activations live on the
// device; the three weight tensors and the bias are read on the host once, in
// PrepareForRun.
typedef paddle::lite::kernels::hip::SparseConvCompute<PRECISION(kFloat), PRECISION(kFloat)> SparseConvHipFp32;
typedef paddle::lite::kernels::hip::SparseConvCompute<PRECISION(kInt8), PRECISION(kFloat)> SparseConvHipInt8Fp32;
typedef paddle::lite::kernels::hip::SparseConvCompute<PRECISION(kInt8), PRECISION(kInt8)> SparseConvHipInt8Int8;

REGISTER_LITE_KERNEL(sparse_conv2d, kHIP, kFloat, kNCHW, SparseConvHipFp32, def)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP))})
    .BindInput("NonZeroWeights", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost))})
    .BindInput("OcNonZeros", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt32))})
    .BindInput("Diffs", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt32))})
    .BindInput("Bias", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost))})
    .BindOutput("Output", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP))})
    .Finalize();

REGISTER_LITE_KERNEL(sparse_conv2d, kHIP, kInt8, kNCHW, SparseConvHipInt8Fp32, int8_fp32_out)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kInt8))})
    .BindInput("NonZeroWeights", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt8))})
    .BindInput("OcNonZeros", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt32))})
    .BindInput("Diffs", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt32))})
    .BindInput("Bias", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kFloat))})
    .BindOutput("Output", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kFloat))})
    .Finalize();

REGISTER_LITE_KERNEL(sparse_conv2d, kHIP, kInt8, kNCHW, SparseConvHipInt8Int8, int8_int8_out)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kInt8))})
    .BindInput("NonZeroWeights", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt8))})
    .BindInput("OcNonZeros", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt32))})
    .BindInput("Diffs", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt32))})
    .BindInput("Bias", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kFloat))})
    .BindOutput("Output", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kInt8))})
    .Finalize();

// lite/kernels/arm/sparse_conv_compute.cc:365-381 (under ENABLE_ARM_FP16).  The
// weight tensors and the bias are the fp32 ones of the pass on the host.
typedef paddle::lite::kernels::hip::SparseConvCompute<PRECISION(kFP16), PRECISION(kFP16)> SparseConvHipFp16;
REGISTER_LITE_KERNEL(sparse_conv2d, kHIP, kFP16, kNCHW, SparseConvHipFp16, def)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kFP16))})
    .BindInput("NonZeroWeights", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kFloat))})
    .BindInput("OcNonZeros", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt32))})
    .BindInput("Diffs", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kInt32))})
    .BindInput("Bias", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kFloat))})
    .BindOutput("Output", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kFP16))})
    .Finalize();
