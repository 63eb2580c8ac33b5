// What the reference's optimiser does around quantised ops, restated for a
// graph of sparse_conv2d and int8 depthwise_conv2d ops that all run on
// TARGET(kHIP) (a variable may have several consumers):
//  * the output-type rule of static_kernel_pick_pass
//    (lite/core/optimizer/mir/static_kernel_pick_pass.cc:97-135): an op with
//    enable_int8 produces int8 only if every consumer of its output has
//    enable_int8 too; its output scale is then the consumer's input scale;
//  * the calib op type_precision_cast_pass puts where a producer's precision
//    differs from what the picked kernel declares
//    (lite/core/optimizer/mir/type_precision_cast_pass.cc);
//  * the io_copy op type_target_cast_pass puts where a tensor lives on
//    another target than the kernel declares
//    (lite/core/optimizer/mir/type_target_cast_pass.cc).
// The result is a list of steps (op description + kernel alias + place) that
// HipProgram runs in order, the counterpart of RuntimeProgram::Run
// (lite/core/program.cc:789-816) for this slice.
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "lite/api/paddle_place.h"
#include "lite/core/kernel.h"
#include "lite/core/op_desc.h"
#include "lite/core/op_lite.h"
#include "lite/core/optimizer/mir/graph.h"
#include "lite/core/scope.h"

namespace paddle {
namespace lite {
namespace mir {

struct ProgramStep {
  OpInfo op;
  std::string kernel;      // "op_type/alias"
  lite_api::Place place;   // place the kernel is created for
};

class Int8ChainPass {
 public:
  // `ops`: sparse_conv2d / depthwise_conv2d ops in execution order (after SparseConvDetectPass).
  // `feeds`: fp32 host tensors in `scope`.  `fetches`: variables wanted back
  // on the host as fp32; the host copy of "v" is named "v/host".
  std::vector<ProgramStep> Apply(const std::vector<OpInfo>& ops, const std::vector<std::string>& feeds, const std::vector<std::string>& fetches, Scope* scope) const;
  // The same on a graph (consumers are read from its links, steps come out in topological order).
  std::vector<ProgramStep> Apply(const Graph& graph, const std::vector<std::string>& feeds, const std::vector<std::string>& fetches, Scope* scope) const;
};

// Creates the op and the kernel of every step once, then launches them in
// order on one stream.
class HipProgram {
 public:
  HipProgram(const std::vector<ProgramStep>& steps, Scope* scope);
  void Run();   // enqueue every step and wait for the stream
  // Enqueues steps [first, last) and returns without waiting: shape check, shape inference and
  // Launch of each, nothing else, so that a caller can time the host side of a step or record
  // the steps into a stream capture.
  void Enqueue(size_t first, size_t last);
  void Sync();  // waits for the stream of the last step
  // Pair launches (lite/kernels/hip/pair_launch.h): an int8 -> int8 sparse_conv2d step followed by the int8 -> int8
  // depthwise_conv2d step that is the only reader of its output runs as one launch where the library says that
  // pays for the step's shapes (from the second Enqueue on: the first one prepares the kernels).  The tensor
  // between the two steps is then not written.  Off by default.
  void set_pair_launch(bool on) { pair_launch_ = on; }
  size_t pairs_joined_last_enqueue() const { return pairs_joined_; }
  size_t size() const { return kernels_.size(); }
  const KernelBase& kernel(size_t i) const { return *kernels_[i]; }

 private:
  std::vector<std::shared_ptr<OpLite>> ops_;
  std::vector<std::unique_ptr<KernelBase>> kernels_;
  std::vector<char> only_reader_is_next_;  // per step: its first output is read by step + 1 and by no other step
  bool pair_launch_ = false;
  size_t pairs_joined_ = 0;
};

}  // namespace mir
}  // namespace lite
}  // namespace paddle
