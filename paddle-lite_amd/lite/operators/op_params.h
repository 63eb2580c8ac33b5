// Parameter bags of the sparse convolution.  Field names, order and defaults
// are the reference's (lite/operators/op_params.h:331-362 ActivationParam,
// :373-400 SparseConvParam) so that kernel code written against the
// reference compiles against this header unchanged.
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "lite/api/paddle_place.h"
#include "lite/core/tensor.h"

namespace paddle {
namespace lite {
namespace operators {

// An empty base as in the reference (lite/operators/op_params.h:36): the
// parameter structs carry no virtual table, their first field sits at offset 0.
struct ParamBase {};

struct ActivationParam : ParamBase {
  const lite::Tensor* X{};
  lite::Tensor* Out{};
  lite_api::ActivationType active_type{lite_api::ActivationType::kIndentity};
  bool has_active{false};
  float Leaky_relu_alpha{0.f};
  float Relu_clipped_coef{6.f};
  std::string Prelu_mode{"channel"};
  lite::Tensor* Prelu_alpha{};
  float Swish_beta{0.f};
  float hard_sigmoid_slope{0.2f};
  float hard_sigmoid_offset{0.5f};
  float hard_swish_threshold{6.0f};
  float hard_swish_scale{6.0f};
  float hard_swish_offset{3.0f};
  float swish_scale{6.0f};
  float relu_threshold{1.0f};
  float Elu_alpha{1.0f};
  float threshold{6.0f};
  bool gelu_approximate{false};
  float softplus_beta{1.0f};
  float softplus_threshold{20.f};
};

struct SparseConvParam : ParamBase {
  const lite::Tensor* x{};
  lite::Tensor* nonzero_weights{};  // nonzero kernel elements
  lite::Tensor* diffs{};            // byte distance between the input channels of successive nonzeros
  lite::Tensor* oc_nonzeros{};      // running nonzero count per output channel
  lite::Tensor* bias{nullptr};
  lite::Tensor* output{};
  int first_ic{0};
  int flag_semi{0};
  std::vector<int> strides{1, 1};
  std::shared_ptr<std::vector<int>> paddings;
  int groups{1};
  std::shared_ptr<std::vector<int>> dilations;
  bool fuse_relu{false};
  ActivationParam activation_param;
  bool enable_int8{false};
  float input_scale{1.0f};
  std::vector<float> weight_scale{};
  float output_scale{1.0f};
  int bit_length{8};
};

// The fields of the reference's ConvParam that the int8 depthwise kernels
// read (lite/operators/op_params.h ConvParam), same names and defaults.
struct ConvParam : ParamBase {
  const lite::Tensor* x{};
  lite::Tensor* filter{};
  lite::Tensor* bias{nullptr};
  lite::Tensor* output{};
  std::vector<int> strides{1, 1};
  std::shared_ptr<std::vector<int>> paddings;
  int groups{1};
  std::shared_ptr<std::vector<int>> dilations;
  bool fuse_relu{false};
  ActivationParam activation_param;
  bool enable_int8{false};
  float input_scale{1.0f};
  std::vector<float> weight_scale{};
  float output_scale{1.0f};
  int bit_length{8};
};

// reference: lite/operators/op_params.h (IoCopyParam)
struct IoCopyParam : ParamBase {
  const lite::Tensor* x{};
  lite::Tensor* y{};
  int process_type{0};
};

// reference: lite/operators/op_params.h:74-78
struct CalibParam : ParamBase {
  const lite::Tensor* input{};
  lite::Tensor* output{};
  float scale{1.0f};
};

}  // namespace operators
}  // namespace lite
}  // namespace paddle
