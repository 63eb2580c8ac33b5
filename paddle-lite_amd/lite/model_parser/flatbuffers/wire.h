// The FlatBuffers binary encoding, as much of it as the model file needs:
// a bounds-checked reader over tables / vectors / strings addressed by
// vtable slot, and a back-to-front builder.  Written against the published
// encoding (little endian; a buffer starts with the 32-bit offset of its root
// table; a table starts with a signed 32-bit offset back to its vtable; a
// vtable is u16 size, u16 table size, then one u16 field offset per slot, 0
// for an absent field; offsets to strings, vectors and tables are unsigned,
// 32 bits, relative to the location that holds them; vectors and strings are
// a u32 element count followed by the elements, strings 0-terminated).
// The reference reads and writes these buffers through flatc-generated
// accessors (lite/model_parser/flatbuffers/*.h over framework.fbs and
// param.fbs); the slot numbers used by the callers of this header follow the
// field order of those schemas.
#pragma once

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace paddle {
namespace lite {
namespace fbs {
namespace wire {

struct FormatError : public std::runtime_error {
  explicit FormatError(const std::string& what) : std::runtime_error(what) {}
};

// ---------------------------------------------------------------- reading
class View {
 public:
  View() = default;
  View(const uint8_t* data, size_t size) : data_(data), size_(size) {}
  const uint8_t* data() const { return data_; }
  size_t size() const { return size_; }

  template <typename T>
  T Read(size_t pos) const {
    Check(pos, sizeof(T));
    T v;
    std::memcpy(&v, data_ + pos, sizeof(T));
    return v;
  }
  // position an unsigned offset stored at `pos` points to
  size_t Indirect(size_t pos) const {
    const size_t target = pos + Read<uint32_t>(pos);
    Check(target, 4);
    return target;
  }
  void Check(size_t pos, size_t len) const {
    if (pos > size_ || len > size_ - pos) throw FormatError("flatbuffer: access outside the buffer");
  }

 private:
  const uint8_t* data_ = nullptr;
  size_t size_ = 0;
};

template <typename T>
class ScalarVector {
 public:
  ScalarVector() = default;
  ScalarVector(const View& v, size_t pos) : view_(v), pos_(pos) {
    n_ = view_.Read<uint32_t>(pos);
    view_.Check(pos + 4, static_cast<size_t>(n_) * sizeof(T));
  }
  size_t size() const { return n_; }
  T operator[](size_t i) const { return view_.Read<T>(pos_ + 4 + i * sizeof(T)); }
  const uint8_t* bytes() const { return n_ ? view_.data() + pos_ + 4 : nullptr; }
  std::vector<T> ToVector() const {
    std::vector<T> out(n_);
    if (n_) std::memcpy(out.data(), bytes(), n_ * sizeof(T));
    return out;
  }

 private:
  View view_;
  size_t pos_ = 0;
  uint32_t n_ = 0;
};

class Table {
 public:
  Table() = default;
  Table(const View& v, size_t pos) : view_(v), pos_(pos), valid_(true) {
    const int32_t back = view_.Read<int32_t>(pos);
    const int64_t vt = static_cast<int64_t>(pos) - back;
    if (vt < 0) throw FormatError("flatbuffer: vtable before the buffer");
    vt_ = static_cast<size_t>(vt);
    vt_size_ = view_.Read<uint16_t>(vt_);
    if (vt_size_ < 4 || (vt_size_ & 1)) throw FormatError("flatbuffer: bad vtable size");
    view_.Check(vt_, vt_size_);
    view_.Check(pos, view_.Read<uint16_t>(vt_ + 2));
  }
  static Table Root(const View& v) { return Table(v, v.Indirect(0)); }
  bool valid() const { return valid_; }

  // position of the field of `slot`, 0 when the field is absent
  size_t Field(int slot) const {
    const size_t entry = 4 + 2 * static_cast<size_t>(slot);
    if (!valid_ || entry + 2 > vt_size_) return 0;
    const uint16_t off = view_.Read<uint16_t>(vt_ + entry);
    return off ? pos_ + off : 0;
  }
  bool Has(int slot) const { return Field(slot) != 0; }
  template <typename T>
  T Scalar(int slot, T def) const {
    const size_t f = Field(slot);
    return f ? view_.Read<T>(f) : def;
  }
  std::string String(int slot) const {
    const size_t f = Field(slot);
    return f ? StringAt(view_, view_.Indirect(f)) : std::string();
  }
  Table Sub(int slot) const {
    const size_t f = Field(slot);
    return f ? Table(view_, view_.Indirect(f)) : Table();
  }
  template <typename T>
  ScalarVector<T> Vector(int slot) const {
    const size_t f = Field(slot);
    return f ? ScalarVector<T>(view_, view_.Indirect(f)) : ScalarVector<T>();
  }
  // vectors of tables / strings: element i is an offset
  size_t VectorSize(int slot) const {
    const size_t f = Field(slot);
    return f ? view_.Read<uint32_t>(view_.Indirect(f)) : 0;
  }
  Table TableAt(int slot, size_t i) const { return Table(view_, ElementTarget(slot, i)); }
  std::string StringAt(int slot, size_t i) const { return StringAt(view_, ElementTarget(slot, i)); }

 private:
  size_t ElementTarget(int slot, size_t i) const {
    const size_t vec = view_.Indirect(Field(slot));
    if (i >= view_.Read<uint32_t>(vec)) throw FormatError("flatbuffer: vector index out of range");
    return view_.Indirect(vec + 4 + 4 * i);
  }
  static std::string StringAt(const View& v, size_t pos) {
    const uint32_t n = v.Read<uint32_t>(pos);
    v.Check(pos + 4, static_cast<size_t>(n) + 1);
    return std::string(reinterpret_cast<const char*>(v.data() + pos + 4), n);
  }

  View view_;
  size_t pos_ = 0, vt_ = 0;
  uint16_t vt_size_ = 0;
  bool valid_ = false;
};

// ---------------------------------------------------------------- writing
// Objects are written from the end of the buffer towards its start, children
// before their parents; an object is named by its distance from the end.
class Builder {
 public:
  using Ref = uint32_t;  // distance of an object's first byte from the end; 0 = none

  Ref CreateString(const std::string& s) {
    PreAlign(s.size() + 1, 4);
    PushBytes("\0", 1);
    PushBytes(s.data(), s.size());
    PushScalar<uint32_t>(static_cast<uint32_t>(s.size()));
    return size();
  }
  template <typename T>
  Ref CreateVector(const T* data, size_t n) {
    PreAlign(n * sizeof(T), 4);
    PreAlign(n * sizeof(T), sizeof(T));
    PushBytes(data, n * sizeof(T));
    PushScalar<uint32_t>(static_cast<uint32_t>(n));
    return size();
  }
  template <typename T>
  Ref CreateVector(const std::vector<T>& v) {
    return CreateVector<T>(v.data(), v.size());
  }
  Ref CreateBoolVector(const std::vector<bool>& v) {
    std::vector<uint8_t> b(v.begin(), v.end());
    return CreateVector<uint8_t>(b);
  }
  // vector of strings or tables
  Ref CreateRefVector(const std::vector<Ref>& refs) {
    PreAlign(refs.size() * 4, 4);
    for (size_t i = refs.size(); i-- > 0;) PushScalar<uint32_t>(ReferTo(refs[i]));
    PushScalar<uint32_t>(static_cast<uint32_t>(refs.size()));
    return size();
  }

  void StartTable() {
    fields_.clear();
    table_end_ = size();
  }
  // Scalars equal to their schema default are left out, as the generated
  // code of the reference does.
  template <typename T>
  void AddScalar(int slot, T v, T def) {
    if (v == def) return;
    PushScalar<T>(v);
    fields_.push_back({slot, size()});
  }
  void AddRef(int slot, Ref r) {
    if (r == 0) return;
    PushScalar<uint32_t>(ReferTo(r));
    fields_.push_back({slot, size()});
  }
  Ref EndTable() {
    PushScalar<int32_t>(0);  // offset to the vtable, patched below
    const uint32_t table = size();
    int slots = 0;
    for (auto& f : fields_) slots = f.slot + 1 > slots ? f.slot + 1 : slots;
    std::vector<uint16_t> vt(2 + static_cast<size_t>(slots), 0);
    vt[0] = static_cast<uint16_t>(2 * vt.size());
    vt[1] = static_cast<uint16_t>(table - table_end_);
    for (auto& f : fields_) vt[2 + f.slot] = static_cast<uint16_t>(table - f.at);
    for (size_t i = vt.size(); i-- > 0;) PushScalar<uint16_t>(vt[i]);
    const int32_t back = static_cast<int32_t>(size() - table);  // vtable lies before the table
    std::memcpy(&buf_[buf_.size() - table], &back, 4);
    return table;
  }

  // Adds the root offset; the finished buffer is data() .. data() + size().
  void Finish(Ref root) {
    PreAlign(4, min_align_);
    PushScalar<uint32_t>(ReferTo(root));
  }
  uint32_t size() const { return used_; }
  const uint8_t* data() const { return buf_.data() + buf_.size() - used_; }
  std::vector<uint8_t> Release() const { return std::vector<uint8_t>(data(), data() + used_); }

 private:
  struct FieldLoc {
    int slot;
    uint32_t at;
  };
  void Grow(size_t more) {
    if (used_ + more <= buf_.size()) return;
    size_t cap = buf_.empty() ? 1024 : buf_.size();
    while (cap < used_ + more) cap *= 2;
    std::vector<uint8_t> bigger(cap, 0);
    if (used_) std::memcpy(bigger.data() + cap - used_, buf_.data() + buf_.size() - used_, used_);
    buf_.swap(bigger);
  }
  void PushBytes(const void* src, size_t n) {
    if (n == 0) return;
    Grow(n);
    used_ += static_cast<uint32_t>(n);
    std::memcpy(&buf_[buf_.size() - used_], src, n);
  }
  void Pad(size_t n) {
    Grow(n);
    for (size_t i = 0; i < n; ++i) buf_[buf_.size() - used_ - 1 - i] = 0;
    used_ += static_cast<uint32_t>(n);
  }
  void Align(size_t a) {
    if (a > min_align_) min_align_ = a;
    Pad((a - used_ % a) % a);
  }
  // pad so that, after `len` more bytes, the size is a multiple of `a`
  void PreAlign(size_t len, size_t a) {
    if (a > min_align_) min_align_ = a;
    Pad((a - (used_ + len) % a) % a);
  }
  template <typename T>
  void PushScalar(T v) {
    Align(sizeof(T));
    PushBytes(&v, sizeof(T));
  }
  // value of an offset field written next that points at `r`
  uint32_t ReferTo(Ref r) {
    Align(4);
    return used_ + 4 - r;
  }

  std::vector<uint8_t> buf_;
  uint32_t used_ = 0;
  size_t min_align_ = 1;
  std::vector<FieldLoc> fields_;
  uint32_t table_end_ = 0;
};

}  // namespace wire
}  // namespace fbs
}  // namespace lite
}  // namespace paddle
