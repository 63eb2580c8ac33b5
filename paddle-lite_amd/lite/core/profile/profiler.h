// What an op and a kernel report to the profiler: the fields of the
// reference's profile::OpCharacter that the sparse_conv2d op and kernel fill
// (lite/core/profile/profiler.h:51-106), with its shape formatting.
#pragma once

#include <string>

#include "lite/core/tensor.h"

namespace paddle {
namespace lite {
namespace profile {

struct OpCharacter {
  std::string op_type{"N/A"};
  std::string kernel_name{"N/A"};
  std::string kernel_func_name{"N/A"};
  std::string remark{"N/A"};
  std::string input_shape{"N/A"};
  std::string output_shape{"N/A"};
  std::string filter_shape{"N/A"};
  float macs{0.f};

  // "2x512x14x14"; "NotImpl" for an empty shape
  static std::string DimToStr(const DDim& dim) {
    if (!dim.size()) return "NotImpl";
    std::string s;
    for (size_t i = 0; i < dim.size(); ++i) {
      s += std::to_string(dim[i]);
      if (i + 1 != dim.size()) s += "x";
    }
    return s;
  }
};

}  // namespace profile
}  // namespace lite
}  // namespace paddle
