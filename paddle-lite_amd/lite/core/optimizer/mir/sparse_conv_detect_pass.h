// sparse_conv_detect_pass: rewrites every eligible conv2d (1x1, stride 1,
// pad 0, group 1, fp32 or int8 weights, enough zeros) of a graph into
// sparse_conv2d and creates its three weight tensors
// (reference: lite/core/optimizer/mir/sparse_conv_detect_pass.{h,cc}, bound
// to TARGET(kARM) only there).
#pragma once

#include <string>
#include <vector>

#include "lite/api/paddle_place.h"
#include "lite/core/op_desc.h"
#include "lite/core/scope.h"

namespace paddle {
namespace lite {
namespace mir {

class Graph;

class SparseConvDetectPass {
 public:
  // reference default 0.6 (lite/api/paddle_api.h:473-474); the predictor
  // passes 1.5 to disable the pass (lite/api/cxx_api_impl.cc:112-123)
  // Any value is accepted here: the predictor passes 1.5 to switch the pass
  // off (reference: lite/api/cxx_api_impl.cc:117-123).
  void SetSparseThreshold(float t) { sparse_threshold_ = t; }
  // The range check of the optimiser tool, which only takes [0, 1]
  // (reference: lite/api/tools/opt_base.cc:78-81).
  static float CheckedToolThreshold(float t) {
    CHECK(t >= 0.f && t <= 1.f) << "Please set sparse_threshold between 0.0 and 1.0.";
    return t;
  }
  float sparse_threshold() const { return sparse_threshold_; }

  // Targets the pass runs for; the reference binds kARM, this build adds kHIP.
  static bool BoundTo(lite_api::TargetType t) { return t == lite_api::TargetType::kARM || t == lite_api::TargetType::kHIP; }

  // The rewrite on the graph, as the reference runs it
  // (sparse_conv_detect_pass.cc:596-857): every eligible conv2d node is
  // replaced by a sparse_conv2d node that takes over its links, the three new
  // weight variables are linked in and the dense filter's node is dropped.
  // Returns how many conv2d ops were replaced.
  int Apply(Graph* graph, Scope* scope) const;
  // Convenience for a list of ops: builds the graph, applies the pass and
  // writes the ops back in topological order (list order for a chain).
  int Apply(std::vector<OpInfo>* ops, Scope* scope) const;

 private:
  float sparse_threshold_{0.6f};
};

}  // namespace mir
}  // namespace lite
}  // namespace paddle
