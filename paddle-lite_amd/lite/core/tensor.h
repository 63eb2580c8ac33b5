// DDim, device-aware Buffer and Tensor: the part of lite::Tensor the sparse
// convolution's op, pass and kernels touch (reference: lite/core/tensor.h,
// lite/core/memory.h, lite/core/target_wrapper.h:118-155).
#pragma once

#include <cstdint>
#include <cstring>
#include <memory>
#include <numeric>
#include <vector>

#include "lite/api/paddle_place.h"
#include "lite/utils/log.h"

namespace paddle {
namespace lite {

using lite_api::DataLayoutType;
using lite_api::Place;
using lite_api::PrecisionType;
using lite_api::TargetType;

class DDim {
 public:
  using value_type = int64_t;
  DDim() = default;
  explicit DDim(const std::vector<value_type>& d) : d_(d) {}
  DDim(std::initializer_list<value_type> d) : d_(d) {}
  value_type operator[](size_t i) const { return d_.at(i); }
  value_type& operator[](size_t i) { return d_.at(i); }
  size_t size() const { return d_.size(); }
  bool empty() const { return d_.empty(); }
  value_type production() const {
    return d_.empty() ? 0 : std::accumulate(d_.begin(), d_.end(), value_type(1), [](value_type a, value_type b) { return a * b; });
  }
  const std::vector<value_type>& Vectorize() const { return d_; }
  bool operator==(const DDim& o) const { return d_ == o.d_; }
  bool operator!=(const DDim& o) const { return d_ != o.d_; }

 private:
  std::vector<value_type> d_;
};

// Raw allocation / copies per target. kHost, kX86 and kARM share the host
// heap (reference: lite/core/memory.cc:25-33); kHIP is device memory.
void* TargetMalloc(TargetType target, size_t size);
void TargetFree(TargetType target, void* data);
enum class IoDirection { HtoH = 0, HtoD, DtoH, DtoD };
// Synchronous copy. stream (a hipStream_t) is used for device copies.
void TargetCopy(IoDirection dir, void* dst, const void* src, size_t size, void* stream = nullptr);

class Buffer {
 public:
  Buffer() = default;
  Buffer(const Buffer&) = delete;
  Buffer& operator=(const Buffer&) = delete;
  ~Buffer() { Free(); }
  void ResetLazy(TargetType target, size_t size) {
    if (target != target_ || size > space_) {
      Free();
      data_ = TargetMalloc(target, size);
      target_ = target;
      space_ = size;
    }
  }
  void Free() {
    if (data_ && space_ > 0) TargetFree(target_, data_);
    data_ = nullptr;
    space_ = 0;
  }
  void* data() const { return data_; }
  size_t space() const { return space_; }
  TargetType target() const { return target_; }

 private:
  void* data_{nullptr};
  size_t space_{0};
  TargetType target_{TargetType::kHost};
};

template <typename T>
struct PrecisionOf;
template <> struct PrecisionOf<float> { static constexpr PrecisionType value = PrecisionType::kFloat; };
template <> struct PrecisionOf<int8_t> { static constexpr PrecisionType value = PrecisionType::kInt8; };
template <> struct PrecisionOf<int32_t> { static constexpr PrecisionType value = PrecisionType::kInt32; };
template <> struct PrecisionOf<uint32_t> { static constexpr PrecisionType value = PrecisionType::kInt32; };
template <> struct PrecisionOf<int64_t> { static constexpr PrecisionType value = PrecisionType::kInt64; };
template <> struct PrecisionOf<uint8_t> { static constexpr PrecisionType value = PrecisionType::kUInt8; };
// binary16 values travel as their bit patterns on the host side
template <> struct PrecisionOf<uint16_t> { static constexpr PrecisionType value = PrecisionType::kFP16; };

using LoD = std::vector<std::vector<uint64_t>>;

class Tensor {
 public:
  Tensor() : buffer_(std::make_shared<Buffer>()) {}

  void Resize(const DDim& d) { dims_ = d; }
  void Resize(const std::vector<int64_t>& d) { dims_ = DDim(d); }
  void Resize(std::initializer_list<int64_t> d) { dims_ = DDim(std::vector<int64_t>(d)); }
  const DDim& dims() const { return dims_; }
  int64_t numel() const { return dims_.production(); }

  template <typename T>
  const T* data() const {
    return static_cast<const T*>(buffer_->data());
  }
  const void* raw_data() const { return buffer_->data(); }

  template <typename T>
  T* mutable_data() {
    return mutable_data<T>(target_);
  }
  template <typename T>
  T* mutable_data(TargetType target) {
    precision_ = PrecisionOf<T>::value;
    return static_cast<T*>(mutable_data(target, static_cast<size_t>(numel()) * sizeof(T)));
  }
  void* mutable_data(TargetType target, size_t bytes) {
    target_ = target;
    memory_size_ = bytes;
    buffer_->ResetLazy(target, bytes);
    return buffer_->data();
  }

  PrecisionType precision() const { return precision_; }
  void set_precision(PrecisionType p) { precision_ = p; }
  TargetType target() const { return target_; }
  bool persistable() const { return persistable_; }
  void set_persistable(bool p) { persistable_ = p; }
  size_t memory_size() const { return memory_size_; }
  const LoD& lod() const { return lod_; }
  void set_lod(const LoD& l) { lod_ = l; }

  // Host-side fill, the counterpart of Tensor::Assign.
  template <typename T>
  void Assign(const T* src, const DDim& d) {
    Resize(d);
    T* dst = mutable_data<T>(TargetType::kHost);
    std::memcpy(dst, src, static_cast<size_t>(numel()) * sizeof(T));
  }

  // Deep copy of data and meta data between any two targets.
  void CopyDataFrom(const Tensor& other, TargetType dst_target, void* stream = nullptr);
  void ShareDataWith(const Tensor& other) {
    buffer_ = other.buffer_;
    dims_ = other.dims_;
    target_ = other.target_;
    precision_ = other.precision_;
    memory_size_ = other.memory_size_;
    lod_ = other.lod_;
  }

 private:
  DDim dims_;
  std::shared_ptr<Buffer> buffer_;
  TargetType target_{TargetType::kHost};
  PrecisionType precision_{PrecisionType::kFloat};
  bool persistable_{false};
  size_t memory_size_{0};
  LoD lod_;
};

}  // namespace lite
}  // namespace paddle
