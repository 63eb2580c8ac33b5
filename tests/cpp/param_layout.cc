// Prints the memory layout (offset and size of every field, size of the
// struct, default values) of SparseConvParam and ActivationParam as declared
// by whichever "lite/operators/op_params.h" the include path finds first: the
// reference's or this repository's.  tests/test_boundary_conformance.py
// compiles it once against each and compares the two printouts.
#include <cstddef>
#include <cstdio>

#include "lite/operators/op_params.h"

using paddle::lite::operators::ActivationParam;
using paddle::lite::operators::SparseConvParam;

// offsetof on a type with a virtual destructor is conditionally supported; both compilers used here support it
#pragma GCC diagnostic ignored "-Winvalid-offsetof"
#define FIELD(S, f) std::printf(#S "." #f " offset %zu size %zu\n", offsetof(S, f), sizeof(static_cast<S*>(nullptr)->f))

int main() {
  std::printf("sizeof(ActivationParam) %zu\n", sizeof(ActivationParam));
  FIELD(ActivationParam, X);
  FIELD(ActivationParam, Out);
  FIELD(ActivationParam, active_type);
  FIELD(ActivationParam, has_active);
  FIELD(ActivationParam, Leaky_relu_alpha);
  FIELD(ActivationParam, Relu_clipped_coef);
  FIELD(ActivationParam, Prelu_mode);
  FIELD(ActivationParam, Prelu_alpha);
  FIELD(ActivationParam, Swish_beta);
  FIELD(ActivationParam, hard_sigmoid_slope);
  FIELD(ActivationParam, hard_sigmoid_offset);
  FIELD(ActivationParam, hard_swish_threshold);
  FIELD(ActivationParam, hard_swish_scale);
  FIELD(ActivationParam, hard_swish_offset);
  FIELD(ActivationParam, swish_scale);
  FIELD(ActivationParam, relu_threshold);
  FIELD(ActivationParam, Elu_alpha);
  FIELD(ActivationParam, threshold);
  FIELD(ActivationParam, gelu_approximate);
  FIELD(ActivationParam, softplus_beta);
  FIELD(ActivationParam, softplus_threshold);
  std::printf("sizeof(SparseConvParam) %zu\n", sizeof(SparseConvParam));
  FIELD(SparseConvParam, x);
  FIELD(SparseConvParam, nonzero_weights);
  FIELD(SparseConvParam, diffs);
  FIELD(SparseConvParam, oc_nonzeros);
  FIELD(SparseConvParam, bias);
  FIELD(SparseConvParam, output);
  FIELD(SparseConvParam, first_ic);
  FIELD(SparseConvParam, flag_semi);
  FIELD(SparseConvParam, strides);
  FIELD(SparseConvParam, paddings);
  FIELD(SparseConvParam, groups);
  FIELD(SparseConvParam, dilations);
  FIELD(SparseConvParam, fuse_relu);
  FIELD(SparseConvParam, activation_param);
  FIELD(SparseConvParam, enable_int8);
  FIELD(SparseConvParam, input_scale);
  FIELD(SparseConvParam, weight_scale);
  FIELD(SparseConvParam, output_scale);
  FIELD(SparseConvParam, bit_length);
  // defaults of a value-initialised parameter
  const SparseConvParam p{};
  std::printf("defaults first_ic %d flag_semi %d strides %zu:%d,%d groups %d fuse_relu %d enable_int8 %d input_scale %g output_scale %g bit_length %d weight_scale %zu paddings %d dilations %d\n", p.first_ic,
              p.flag_semi, p.strides.size(), p.strides[0], p.strides[1], p.groups, p.fuse_relu, p.enable_int8, p.input_scale, p.output_scale, p.bit_length, p.weight_scale.size(), p.paddings ? 1 : 0,
              p.dilations ? 1 : 0);
  const ActivationParam& a = p.activation_param;
  std::printf("defaults active_type %d has_active %d Leaky_relu_alpha %g Relu_clipped_coef %g Prelu_mode %s hard_sigmoid %g %g hard_swish %g %g %g swish_scale %g relu_threshold %g Elu_alpha %g threshold %g gelu %d softplus %g %g\n",
              static_cast<int>(a.active_type), a.has_active, a.Leaky_relu_alpha, a.Relu_clipped_coef, a.Prelu_mode.c_str(), a.hard_sigmoid_slope, a.hard_sigmoid_offset, a.hard_swish_threshold, a.hard_swish_scale,
              a.hard_swish_offset, a.swish_scale, a.relu_threshold, a.Elu_alpha, a.threshold, a.gelu_approximate, a.softplus_beta, a.softplus_threshold);
  return 0;
}
