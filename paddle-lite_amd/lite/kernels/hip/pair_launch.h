// Two steps as one launch.  No counterpart in the reference, where RuntimeProgram::Run launches every
// instruction on its own (lite/core/program.cc:789-816): the library can run an int8 -> int8 sparse_conv2d
// and the int8 -> int8 depthwise_conv2d behind it in one kernel (pl_sparse_conv_dwconv3x3_run).  A kernel
// class that can be one end of such a pair implements this interface; mir::HipProgram asks both ends and joins
// them when the tensor between them has no other reader and the library says the one launch pays.
#pragma once

namespace paddle {
namespace lite {
namespace kernels {
namespace hip {

struct PairEndpoint {
  void* handle = nullptr;   // pl_sparse_conv_handle* (first) or pl_dwconv_handle* (second)
  const void* x = nullptr;  // input on the device
  void* out = nullptr;      // output on the device (allocated for the shape InferShape has set)
  int batch = 0, h = 0, w = 0;  // input shape (NCHW)
  void* stream = nullptr;
};

class PairLaunch {
 public:
  virtual ~PairLaunch() = default;
  enum Role { kFirst = 1, kSecond = 2 };  // the int8 -> int8 pointwise layer, the int8 -> int8 depthwise layer
  virtual Role pair_role() const = 0;
  // Fills `e` for the shapes the op has inferred; false before the kernel's first Launch (no handle yet).
  virtual bool pair_endpoint(PairEndpoint* e) = 0;
};

}  // namespace hip
}  // namespace kernels
}  // namespace lite
}  // namespace paddle
