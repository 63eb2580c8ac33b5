// calib kernels of TARGET(kHIP): fp32 -> int8 and int8 -> fp32 with a
// per-tensor scale, device to device
// (reference: lite/kernels/arm/calib_compute.cc:31-38, :60-68 and the
// registrations at :186-330, aliases fp32_to_int8 / int8_to_fp32).
#include "lite/core/op_registry.h"
#include "lite/operators/op_params.h"
#include "pl_sparse_conv.h"

namespace paddle {
namespace lite {
namespace kernels {
namespace hip {

class CalibComputeFp32ToInt8 : public KernelLite<TARGET(kHIP), PRECISION(kInt8)> {
 public:
  using param_t = operators::CalibParam;
  void Run() override {
    auto& param = this->Param<param_t>();
    CHECK(param.input->target() == TargetType::kHIP) << "calib fp32_to_int8: input is not on the device";
    const float* din = static_cast<const float*>(param.input->raw_data());
    int8_t* dout = param.output->mutable_data<int8_t>(TargetType::kHIP);
    const int rc = pl_calib_fp32_to_int8(din, dout, param.input->numel(), param.scale, this->ctx_->As<HIPContext>().stream());
    if (rc != PL_OK) LOG(FATAL) << "calib fp32_to_int8: " << pl_last_error();
  }
};

class CalibComputeInt8ToFp32 : public KernelLite<TARGET(kHIP), PRECISION(kInt8)> {
 public:
  using param_t = operators::CalibParam;
  void Run() override {
    auto& param = this->Param<param_t>();
    CHECK(param.input->target() == TargetType::kHIP) << "calib int8_to_fp32: input is not on the device";
    const int8_t* din = static_cast<const int8_t*>(param.input->raw_data());
    float* dout = param.output->mutable_data<float>(TargetType::kHIP);
    const int rc = pl_calib_int8_to_fp32(din, dout, param.input->numel(), param.scale, this->ctx_->As<HIPContext>().stream());
    if (rc != PL_OK) LOG(FATAL) << "calib int8_to_fp32: " << pl_last_error();
  }
};

}  // namespace hip
}  // namespace kernels
}  // namespace lite
}  // namespace paddle

REGISTER_LITE_KERNEL(calib, kHIP, kInt8, kNCHW, paddle::lite::kernels::hip::CalibComputeFp32ToInt8, fp32_to_int8)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kFloat))})
    .BindOutput("Out", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kInt8))})
    .Finalize();

REGISTER_LITE_KERNEL(calib, kHIP, kInt8, kNCHW, paddle::lite::kernels::hip::CalibComputeInt8ToFp32, int8_to_fp32)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kInt8))})
    .BindOutput("Out", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kFloat))})
    .Finalize();
