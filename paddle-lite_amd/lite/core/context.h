// Per-kernel execution context.  A HIP kernel needs exactly one thing from
// it: the stream its work is enqueued on (reference pattern:
// lite/core/context.h:294-347 ARMContext, :408-420 KernelContext::As<T>()).
#pragma once

#include <memory>

#include "lite/api/paddle_place.h"
#include "lite/utils/log.h"

namespace paddle {
namespace lite {

class HostContext {};

// Context of TARGET(kHIP): device ordinal and hipStream_t (kept as void* so
// that this header needs no HIP include).
class HIPContext {
 public:
  void Init(int device = 0, void* stream = nullptr) {
    device_ = device;
    stream_ = stream;
  }
  int device() const { return device_; }
  void* stream() const { return stream_; }
  void SetStream(void* s) { stream_ = s; }
  // Blocks until everything enqueued on the stream has finished.
  void Sync() const;

 private:
  int device_{0};
  void* stream_{nullptr};
};

class KernelContext {
 public:
  template <typename ContextT>
  ContextT& As() {
    return Slot<ContextT>();
  }

 private:
  template <typename ContextT>
  ContextT& Slot();
  std::unique_ptr<HostContext> host_;
  std::unique_ptr<HIPContext> hip_;
};

template <>
inline HostContext& KernelContext::Slot<HostContext>() {
  if (!host_) host_.reset(new HostContext);
  return *host_;
}
template <>
inline HIPContext& KernelContext::Slot<HIPContext>() {
  if (!hip_) hip_.reset(new HIPContext);
  return *hip_;
}

// reference: lite/core/context.h:423-486 (ContextScheduler::NewContext)
class ContextScheduler {
 public:
  static ContextScheduler& Global() {
    static ContextScheduler s;
    return s;
  }
  std::unique_ptr<KernelContext> NewContext(lite_api::TargetType target) {
    std::unique_ptr<KernelContext> ctx(new KernelContext);
    if (target == lite_api::TargetType::kHIP) {
      ctx->As<HIPContext>().Init(0, default_stream_);
    } else {
      ctx->As<HostContext>();
    }
    return ctx;
  }
  void SetDefaultHIPStream(void* s) { default_stream_ = s; }

 private:
  void* default_stream_{nullptr};
};

}  // namespace lite
}  // namespace paddle
