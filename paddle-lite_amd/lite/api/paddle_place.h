// Target / precision / layout / activation enums and Place, with the values of
// the reference (lite/api/paddle_place.h:45-149) plus one new target: kHIP.
#pragma once

#include <string>

namespace paddle {
namespace lite_api {

enum class TargetType : int {
  kUnk = 0, kHost = 1, kX86 = 2, kCUDA = 3, kARM = 4, kOpenCL = 5, kAny = 6, kFPGA = 7, kNPU = 8, kXPU = 9,
  kBM = 10, kMLU = 11, kRKNPU = 12, kAPU = 13, kHuaweiAscendNPU = 14, kImaginationNNA = 15, kIntelFPGA = 16,
  kMetal = 17, kNNAdapter = 18,
  kHIP = 19,  // AMD Instinct (gfx950) through HIP; appended so existing values keep their meaning
  NUM = 20,
};

enum class PrecisionType : int {
  kUnk = 0, kFloat = 1, kInt8 = 2, kInt32 = 3, kAny = 4, kFP16 = 5, kBool = 6, kInt64 = 7, kInt16 = 8, kUInt8 = 9, kFP64 = 10, NUM = 11,
};

enum class DataLayoutType : int {
  kUnk = 0, kNCHW = 1, kAny = 2, kNHWC = 3, kImageDefault = 4, kImageFolder = 5, kImageNW = 6, kMetalTexture2DArray = 7, kMetalTexture2D = 8, NUM = 9,
};

// Only the members the sparse convolution can meet are listed by name; the
// numeric values are the reference's.
enum class ActivationType : int {
  kIndentity = 0, kRelu = 1, kRelu6 = 2, kPRelu = 3, kLeakyRelu = 4, kSigmoid = 5, kTanh = 6, kSwish = 7, kExp = 8, kAbs = 9,
  kHardSwish = 10, kReciprocal = 11, kThresholdedRelu = 12, kElu = 13, kHardSigmoid = 14, kLog = 15, kSigmoid_v2 = 16, kTanh_v2 = 17,
  kGelu = 18, kErf = 19, kSign = 20, kSoftPlus = 21, kMish = 22, kSilu = 23, kLog1p = 24, NUM = 25,
};

inline const char* TargetToStr(TargetType t) {
  static const char* names[] = {"unk", "host", "x86", "cuda", "arm", "opencl", "any", "fpga", "npu", "xpu", "bm", "mlu", "rknpu", "apu", "huawei_ascend_npu", "imagination_nna", "intel_fpga", "metal", "nnadapter", "hip"};
  int i = static_cast<int>(t);
  return (i >= 0 && i < static_cast<int>(TargetType::NUM)) ? names[i] : "unk";
}

inline const char* PrecisionToStr(PrecisionType p) {
  static const char* names[] = {"unk", "float", "int8_t", "int32_t", "any", "float16", "bool", "int64_t", "int16_t", "uint8_t", "double"};
  int i = static_cast<int>(p);
  return (i >= 0 && i < static_cast<int>(PrecisionType::NUM)) ? names[i] : "unk";
}

struct Place {
  TargetType target{TargetType::kUnk};
  PrecisionType precision{PrecisionType::kUnk};
  DataLayoutType layout{DataLayoutType::kUnk};
  int16_t device{0};

  Place() = default;
  Place(TargetType t, PrecisionType p = PrecisionType::kFloat, DataLayoutType l = DataLayoutType::kNCHW, int16_t d = 0) : target(t), precision(p), layout(l), device(d) {}
  bool operator==(const Place& o) const { return target == o.target && precision == o.precision && layout == o.layout && device == o.device; }
  bool operator!=(const Place& o) const { return !(*this == o); }
  std::string DebugString() const { return std::string(TargetToStr(target)) + "/" + PrecisionToStr(precision); }
};

}  // namespace lite_api
}  // namespace paddle

#define TARGET(item__) paddle::lite_api::TargetType::item__
#define PRECISION(item__) paddle::lite_api::PrecisionType::item__
#define DATALAYOUT(item__) paddle::lite_api::DataLayoutType::item__
