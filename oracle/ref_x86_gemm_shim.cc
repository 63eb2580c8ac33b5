// Thin C entry point around the reference's own x86 int8 GEMM, driven the way
// its dense conv2d kernel drives it for a 1x1 / stride 1 / pad 0 convolution.
// Compiled from the sources where they lie in the reference checkout (never
// copied); built only where that checkout is present, output in oracle/_ref/.
// TEST INFRASTRUCTURE ONLY: the "x86 dense conv2d 1x1" leg of the CPU
// baseline.  A timing comparator, not a checker: the GEMM biases activations
// to unsigned and sums pairs of products in saturating 16-bit arithmetic
// (lite/backends/x86/math/gemm_s8u8_kernel.cc:123-129), which is exact for
// the small inputs of the reference's own test and not for the full int8 range.
//
// reference: lite/kernels/x86/conv_compute.cc:215-289 (PrepareForRun: one
//            generate_gemm_s8u8_x86_kern<float> per group, M = output
//            channels, N = H*W, K = input channels, Sa = per-channel weight
//            scales, Sb = input scale, relu_type 0 none / 1 relu / 2 relu6 /
//            3 leaky_relu), :291-340 (Run: one compute() per image, serial)
#include <chrono>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <cstdint>
#include <memory>
#include <vector>

#include "lite/backends/x86/math/gemm_s8u8_compute.h"

extern "C" {

// Runs `reps` passes over the batch and returns the seconds spent in the
// compute() calls (construction, which packs the weights, is outside, as
// PrepareForRun is outside Run).  threads = 1 is the reference's serial loop
// over images; threads > 1 deals the images to OpenMP threads, each with its
// own GEMM object (an extension for an all-cores figure).
double ref_x86_conv1x1_s8_f32(const int8_t* x, float* out, int num, int chout,
                              int hw, int chin, const int8_t* weights,
                              const float* weight_scale, float input_scale,
                              const float* bias, int relu_type,
                              float relu_alpha, int reps, int threads) {
  using Gemm = paddle::lite::x86::math::generate_gemm_s8u8_x86_kern<float>;
  if (threads < 1) threads = 1;
  std::vector<std::unique_ptr<Gemm>> gemm(threads);
  for (int t = 0; t < threads; ++t)
    gemm[t].reset(new Gemm(false, false, chout, hw, chin, weights, hw,
                           weight_scale, input_scale, 1.f, bias, relu_type,
                           relu_alpha));
  const auto t0 = std::chrono::steady_clock::now();
  for (int r = 0; r < reps; ++r) {
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int b = 0; b < num; ++b) {
      int t = 0;
#ifdef _OPENMP
      t = omp_get_thread_num();
#endif
      gemm[t]->compute(weights, x + static_cast<int64_t>(b) * chin * hw,
                       out + static_cast<int64_t>(b) * chout * hw);
    }
  }
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0)
      .count();
}

}  // extern "C"
