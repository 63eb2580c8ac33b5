// io_copy kernels of TARGET(kHIP): host -> device and device -> host, in the
// pattern of the other device targets
// (reference: lite/kernels/xpu/io_copy_compute.cc:52-115).
#include "lite/core/op_registry.h"
#include "lite/operators/op_params.h"

namespace paddle {
namespace lite {
namespace kernels {
namespace hip {

class IoCopyHostToHipCompute : public KernelLite<TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny)> {
 public:
  void Run() override {
    auto& param = this->Param<operators::IoCopyParam>();
    CHECK(param.x->target() != TargetType::kHIP) << "io_copy host_to_device: input is already on the device";
    param.y->CopyDataFrom(*param.x, TargetType::kHIP, this->ctx_->As<HIPContext>().stream());
  }
};

class IoCopyHipToHostCompute : public KernelLite<TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny)> {
 public:
  void Run() override {
    auto& param = this->Param<operators::IoCopyParam>();
    CHECK(param.x->target() == TargetType::kHIP) << "io_copy device_to_host: input is not on the device";
    param.y->CopyDataFrom(*param.x, TargetType::kHost, this->ctx_->As<HIPContext>().stream());
  }
};

}  // namespace hip
}  // namespace kernels
}  // namespace lite
}  // namespace paddle

REGISTER_LITE_KERNEL(io_copy, kHIP, kAny, kAny, paddle::lite::kernels::hip::IoCopyHostToHipCompute, host_to_device)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kAny), DATALAYOUT(kAny))})
    .BindOutput("Out", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny))})
    .Finalize();

REGISTER_LITE_KERNEL(io_copy, kHIP, kAny, kAny, paddle::lite::kernels::hip::IoCopyHipToHostCompute, device_to_host)
    .BindInput("Input", {paddle::lite::LiteType::GetTensorTy(TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny))})
    .BindOutput("Out", {paddle::lite::LiteType::GetTensorTy(TARGET(kHost), PRECISION(kAny), DATALAYOUT(kAny))})
    .Finalize();
