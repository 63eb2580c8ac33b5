#include "lite/core/tensor.h"

#include <hip/hip_runtime_api.h>

#include <cstdlib>

#include "lite/core/context.h"

namespace paddle {
namespace lite {

namespace {
bool IsHostLike(TargetType t) { return t == TargetType::kHost || t == TargetType::kX86 || t == TargetType::kARM; }

void CheckHip(hipError_t e, const char* what) {
  if (e != hipSuccess) LOG(FATAL) << what << ": " << hipGetErrorString(e);
}
}  // namespace

void* TargetMalloc(TargetType target, size_t size) {
  if (size == 0) size = 16;
  if (IsHostLike(target)) {
    void* p = nullptr;
    if (posix_memalign(&p, 64, size) != 0) LOG(FATAL) << "host allocation of " << size << " bytes failed";
    return p;
  }
  if (target == TargetType::kHIP) {
    void* p = nullptr;
    CheckHip(hipMalloc(&p, size), "hipMalloc");
    return p;
  }
  LOG(FATAL) << "TargetMalloc: unsupported target " << lite_api::TargetToStr(target);
  return nullptr;
}

void TargetFree(TargetType target, void* data) {
  if (!data) return;
  if (IsHostLike(target)) {
    free(data);
  } else if (target == TargetType::kHIP) {
    (void)hipFree(data);
  }
}

void TargetCopy(IoDirection dir, void* dst, const void* src, size_t size, void* stream) {
  if (size == 0) return;
  if (dir == IoDirection::HtoH) {
    std::memcpy(dst, src, size);
    return;
  }
  const hipMemcpyKind kind = dir == IoDirection::HtoD ? hipMemcpyHostToDevice : dir == IoDirection::DtoH ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice;
  hipStream_t s = static_cast<hipStream_t>(stream);
  CheckHip(hipMemcpyAsync(dst, src, size, kind, s), "hipMemcpyAsync");
  CheckHip(hipStreamSynchronize(s), "hipStreamSynchronize");
}

void Tensor::CopyDataFrom(const Tensor& other, TargetType dst_target, void* stream) {
  dims_ = other.dims_;
  precision_ = other.precision_;
  lod_ = other.lod_;
  const size_t bytes = other.memory_size_;
  void* dst = mutable_data(dst_target, bytes);
  const bool src_dev = other.target_ == TargetType::kHIP, dst_dev = dst_target == TargetType::kHIP;
  const IoDirection dir = src_dev ? (dst_dev ? IoDirection::DtoD : IoDirection::DtoH) : (dst_dev ? IoDirection::HtoD : IoDirection::HtoH);
  TargetCopy(dir, dst, other.raw_data(), bytes, stream);
}

void HIPContext::Sync() const { CheckHip(hipStreamSynchronize(static_cast<hipStream_t>(stream_)), "hipStreamSynchronize"); }

}  // namespace lite
}  // namespace paddle
