// Thin C entry points around the reference's own naive test math, compiled
// from the header where it lies in the reference checkout (never copied).
// Built only where that checkout is present; output goes to oracle/_ref/.
// TEST INFRASTRUCTURE ONLY: used to validate the restated oracle and as the
// "reference" CPU baseline.
//
// reference: lite/tests/utils/naive_math_impl.h:246-331 (basic_gemm),
//            lite/tests/utils/naive_math_impl.h:395-519 (conv_basic)
#include <cstdint>
#include <cstdio>

#include "lite/tests/utils/naive_math_impl.h"

extern "C" {

// C[m x n] = act(A[m x k] * B[k x n] + bias), called like the sparse tests do
// (no transposes, alpha 1, beta 0).
void ref_basic_gemm_f32(int m, int n, int k, const float* a, const float* b,
                        float* c, const float* bias, int flag_bias,
                        int flag_act, float six, float leaky_alpha,
                        float hs_scale, float hs_offset, float hs_threshold) {
  basic_gemm<float, float>(false, false, m, n, k, 1.f, a, k, b, n, 0.f, c, n,
                           bias, flag_bias != 0, flag_act, six, leaky_alpha,
                           hs_scale, hs_offset, hs_threshold);
}

// 1x1 / stride 1 / pad 0 / group 1 convolution over a batch, fp32.
void ref_conv1x1_f32(const float* x, float* out, int num, int chout, int h,
                     int w, int chin, const float* weights, const float* bias,
                     int flag_bias, int act_type, float six, float leaky_alpha,
                     float hs_scale, float hs_offset, float hs_threshold) {
  conv_basic<float, float>(x, out, num, chout, h, w, chin, h, w, weights, bias,
                           1, 1, 1, 1, 1, 1, 1, 0, 0, flag_bias != 0, act_type,
                           six, leaky_alpha, hs_scale, hs_offset,
                           hs_threshold);
}

// Same, int8 inputs with int32 accumulators (no bias, no activation): the
// exact integer sums the int8 kernels must reproduce.
void ref_conv1x1_s8_s32(const int8_t* x, int32_t* out, int num, int chout,
                        int h, int w, int chin, const int8_t* weights) {
  conv_basic<int8_t, int32_t>(x, out, num, chout, h, w, chin, h, w, weights,
                              nullptr, 1, 1, 1, 1, 1, 1, 1, 0, 0, false, 0);
}

// Depthwise 3x3 (group == channels), int8 inputs, int32 accumulators.
void ref_dwconv3x3_s8_s32(const int8_t* x, int32_t* out, int num, int ch,
                          int hout, int wout, int hin, int win,
                          const int8_t* weights, int stride, int pad) {
  conv_basic<int8_t, int32_t>(x, out, num, ch, hout, wout, ch, hin, win,
                              weights, nullptr, ch, 3, 3, stride, stride, 1, 1,
                              pad, pad, false, 0);
}

}  // extern "C"
