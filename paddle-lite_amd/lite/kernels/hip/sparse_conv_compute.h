// sparse_conv2d kernels of TARGET(kHIP): the class the reference has for
// TARGET(kARM) (lite/kernels/arm/sparse_conv_compute.h:25-50), with the
// gfx950 library behind Run().
#pragma once

#include <string>
#include <vector>

#include "lite/core/kernel.h"
#include "lite/core/profile/profiler.h"
#include "lite/kernels/hip/pair_launch.h"
#include "lite/operators/op_params.h"

struct pl_sparse_conv_handle;

namespace paddle {
namespace lite {
namespace kernels {
namespace hip {

template <PrecisionType Ptype, PrecisionType OutType>
class SparseConvCompute : public KernelLite<TARGET(kHIP), Ptype>, public PairLaunch {
 public:
  using param_t = operators::SparseConvParam;
  ~SparseConvCompute() override;

  void PrepareForRun() override;
  // Nothing to redo when shapes change: the library keeps channel indices,
  // not byte offsets, so any batch and spatial size can follow.
  void ReInitWhenNeeded() override {}
  void Run() override;

  const std::vector<float>& merged_scales() const { return w_scale_; }

  // First end of a pair launch (pair_launch.h): only the int8 -> int8 kernel can be one.
  PairLaunch::Role pair_role() const override { return PairLaunch::kFirst; }
  bool pair_endpoint(PairEndpoint* e) override;

  // The math entry point and algorithm of the last Run(), for the profiler
  // (the ARM class reports "sparse_conv_fp32_pipelined" etc. through
  // KERNEL_FUNC_NAME, lite/kernels/arm/sparse_conv_compute.h:34-43, compiled
  // in under LITE_WITH_PROFILE only).  Run() only remembers the call's shape;
  // the name is put together here, when a profiler asks
  // (lite/core/program.cc:789-816 asks after the kernel has run).
  void SetProfileRuntimeKernelInfo(paddle::lite::profile::OpCharacter* ch) const { ch->kernel_func_name = kernel_func_name(); }
  std::string kernel_func_name() const;

 private:
  void Upload(int kind);

  Tensor bias_;
  bool flag_trans_bias_{false};
  std::vector<float> w_scale_;
  pl_sparse_conv_handle* handle_{nullptr};
  int64_t ic_{0};  // input channels the weights were prepared for
  int last_batch_{-1}, last_im_size_{-1};  // shape of the last Run(); -1 before the first
};

// The reference divides the int8-output leaky_relu slope by the output scale
// (lite/kernels/arm/sparse_conv_compute.cc:86-90) and scales the hard_swish
// offset / threshold twice (:91-100 and again in
// lite/backends/arm/math/sparse_conv_impl.cc:3713-3720).  true (default)
// reproduces that; false scales once and leaves the slope alone.
void SetSparseConvReferenceQuirks(bool on);
bool SparseConvReferenceQuirks();

}  // namespace hip
}  // namespace kernels
}  // namespace lite
}  // namespace paddle
