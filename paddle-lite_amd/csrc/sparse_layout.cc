#include "sparse_layout.h"

#include <cstring>

namespace pl {

namespace {

template <typename T>
inline bool NonZero(T v) {
  return v != static_cast<T>(0);
}

// Emits index entries for a stream of nonzeros: the byte distance to the
// next entry, and after every row the running total in the row's last slot.
class DiffWriter {
 public:
  DiffWriter(int32_t* diffs, int bytes_per_channel)
      : diffs_(diffs), step_(bytes_per_channel) {}

  // Registers an entry at input channel `c` stored in slot `slot`.
  void Entry(int c, uint32_t slot) {
    if (have_) {
      diffs_[prev_slot_] = (c - prev_c_) * step_;
    } else {
      first_c_ = c;
    }
    have_ = true;
    prev_c_ = c;
    prev_slot_ = slot;
  }
  int first_ic() const { return have_ ? first_c_ : 0; }
  // Offset of the wrap from the last entry back to the first one.
  int32_t WrapDiff() const { return (first_c_ - prev_c_) * step_; }
  bool any() const { return have_; }
  uint32_t last_slot() const { return prev_slot_; }

 private:
  int32_t* diffs_;
  int step_;
  bool have_ = false;
  int first_c_ = 0, prev_c_ = 0;
  uint32_t prev_slot_ = 0;
};

// Replace the slot before each row end by the sum of everything up to it.
void PrefixIntoRowEnds(int32_t* diffs, const uint32_t* ends, int n) {
  int32_t sum = 0;
  uint32_t i = 0;
  for (int r = 0; r < n; ++r) {
    while (i < ends[r]) sum += diffs[i++];
    if (i) diffs[i - 1] = sum;
  }
}

}  // namespace

template <typename T>
SemiCounts CountSemi(const T* w, int oc, int ic) {
  SemiCounts c;
  const int even = oc - (oc & 1);
  int64_t in_pairs = 0, blocks = 0, tail = 0;
  for (int r = 0; r < even; r += 2) {
    const T* a = w + static_cast<size_t>(r) * ic;
    const T* b = a + ic;
    for (int k = 0; k < ic; ++k) {
      const int na = NonZero(a[k]), nb = NonZero(b[k]);
      in_pairs += na + nb;
      blocks += (na | nb);
    }
  }
  for (int r = even; r < oc; ++r)
    for (int k = 0; k < ic; ++k) tail += NonZero(w[static_cast<size_t>(r) * ic + k]);
  c.count_channels = oc;
  c.count_nonzeroes = c.count_blocks = static_cast<int>(in_pairs + tail);
  // at least 1.8 nonzeros per non-empty 2x1 block
  if (in_pairs * 5 >= blocks * 9) {
    c.flag_semi = 1;
    c.count_channels = oc / 2 + oc % 2;
    c.count_nonzeroes = static_cast<int>(2 * blocks + tail);
    c.count_blocks = static_cast<int>(blocks + tail);
  }
  c.zeros = oc * ic - c.count_nonzeroes;
  return c;
}

template <typename T>
int CountZerosPad4(const T* w, int oc, int ic, int* num_build_nonzeroes) {
  int real = 0, padded = 0;
  for (int r = 0; r < oc; ++r) {
    int n = 0;
    for (int k = 0; k < ic; ++k) n += NonZero(w[static_cast<size_t>(r) * ic + k]);
    real += n;
    padded += (n + 3) / 4 * 4;
  }
  *num_build_nonzeroes = padded;
  return oc * ic - real;
}

template <typename T>
int PackWeights(const T* w, int oc, int ic, int im_size, bool semi, T* nz,
                uint32_t* ends, int32_t* diffs) {
  const bool pad4 = !semi && sizeof(T) == 4;  // fp32 unstructured only
  DiffWriter dw(diffs, static_cast<int>(sizeof(T)) * im_size);
  uint32_t slot = 0;   // index entry being written
  uint32_t wpos = 0;   // weight being written
  int n_ends = 0;
  const int even = semi ? oc - (oc & 1) : 0;
  for (int r = 0; r < even; r += 2) {
    const T* a = w + static_cast<size_t>(r) * ic;
    const T* b = a + ic;
    for (int k = 0; k < ic; ++k) {
      if (!(NonZero(a[k]) || NonZero(b[k]))) continue;
      nz[wpos++] = a[k];
      nz[wpos++] = b[k];
      dw.Entry(k, slot++);
    }
    ends[n_ends++] = slot;
  }
  for (int r = even; r < oc; ++r) {
    const T* a = w + static_cast<size_t>(r) * ic;
    const uint32_t begin = slot;
    for (int k = 0; k < ic; ++k) {
      if (!NonZero(a[k])) continue;
      nz[wpos++] = a[k];
      dw.Entry(k, slot++);
    }
    ends[n_ends++] = slot;
    if (pad4) {
      for (uint32_t n = slot - begin; n & 3u; ++n) {
        nz[wpos++] = static_cast<T>(0);
        diffs[slot++] = 0;
      }
    }
  }
  if (!dw.any()) return 0;
  if (pad4) {
    // the wrap entry takes part in the running sums
    diffs[dw.last_slot()] = dw.WrapDiff();
    PrefixIntoRowEnds(diffs, ends, n_ends);
  } else {
    // the wrap entry is stored after the running sums were formed
    diffs[dw.last_slot()] = 0;
    PrefixIntoRowEnds(diffs, ends, n_ends);
    diffs[dw.last_slot()] = dw.WrapDiff();
  }
  return dw.first_ic();
}

bool DecodeLayout(WeightType type, bool semi, const void* nonzero_weights,
                  int64_t n_weights, const uint32_t* ends, const int32_t* diffs,
                  int64_t n_diffs, int first_ic, int oc, int ic, int im_size,
                  DecodedLayout* out, std::string* error) {
  auto fail = [&](const std::string& msg) {
    if (error) *error = msg;
    return false;
  };
  if (oc <= 0 || ic <= 0 || im_size <= 0) return fail("oc, ic and im_size must be positive");
  if (first_ic < 0 || first_ic >= ic) return fail("first_ic outside [0, ic)");
  if (n_weights < 0 || n_diffs < 0) return fail("negative array length");
  const int esize = type == WeightType::kFloat ? 4 : 1;
  const int64_t step = static_cast<int64_t>(esize) * im_size;
  const bool pad4 = !semi && type == WeightType::kFloat;
  const int pairs = semi ? oc / 2 : 0;
  const int n_groups = semi ? pairs + (oc & 1) : oc;

  out->oc = oc;
  out->ic = ic;
  out->semi = semi;
  out->type = type;
  out->groups.clear();
  out->ic_index.clear();
  out->w0.clear();
  out->w1.clear();
  out->nnz = 0;
  out->stored_weights = 0;

  auto weight_bits = [&](int64_t i) -> uint32_t {
    if (type == WeightType::kFloat) {
      uint32_t b;
      std::memcpy(&b, static_cast<const float*>(nonzero_weights) + i, 4);
      return b;
    }
    return static_cast<uint32_t>(static_cast<int32_t>(static_cast<const int8_t*>(nonzero_weights)[i]));
  };
  auto is_zero_bits = [&](uint32_t b) {
    return type == WeightType::kFloat ? (b << 1) == 0 : b == 0;
  };

  uint32_t prev_end = 0;
  for (int g = 0; g < n_groups; ++g) {
    const uint32_t end = ends[g];
    if (end < prev_end) return fail("OcNonZeros is not monotone");
    uint32_t begin = prev_end;
    if (pad4 && g > 0 && (prev_end & 3u)) begin = prev_end + (4u - (prev_end & 3u));
    if (begin > end) {
      // an empty row after a padded one: its end equals the padded start
      return fail("OcNonZeros row end lies inside the previous row's padding");
    }
    if (static_cast<int64_t>(end) > n_diffs) return fail("OcNonZeros exceeds the Diffs length");
    const bool pair = semi && g < pairs;
    RowGroup rg;
    rg.row0 = semi ? (pair ? 2 * g : 2 * pairs) : g;
    rg.nrows = pair ? 2 : 1;
    rg.first = static_cast<uint32_t>(out->ic_index.size());
    rg.count = end - begin;
    // byte offset of this row's first activation relative to first_ic
    int64_t off = (g == 0 || prev_end == 0) ? 0 : diffs[prev_end - 1];
    // weights: pairs are stored interleaved; the odd tail row of a semi
    // layout continues right after the last pair
    const int64_t wbase = semi ? (pair ? 2 * static_cast<int64_t>(begin)
                                       : 2 * static_cast<int64_t>(prev_end))
                               : static_cast<int64_t>(begin);
    const int64_t wcount = pair ? 2 * static_cast<int64_t>(rg.count) : rg.count;
    if (wbase + wcount > n_weights) return fail("NonZeroWeights is shorter than OcNonZeros implies");
    int last_c = -1;
    for (uint32_t j = 0; j < rg.count; ++j) {
      if (off % step != 0) return fail("Diffs entry is not a multiple of sizeof(T)*im_size");
      const int64_t c = first_ic + off / step;
      if (c < 0 || c >= ic) return fail("Diffs walk leaves the input channels");
      if (static_cast<int>(c) <= last_c) return fail("input channels of a row are not increasing");
      last_c = static_cast<int>(c);
      out->ic_index.push_back(static_cast<uint32_t>(c));
      uint32_t a = weight_bits(pair ? wbase + 2 * j : wbase + j);
      uint32_t b = pair ? weight_bits(wbase + 2 * j + 1) : 0u;
      out->w0.push_back(a);
      out->w1.push_back(b);
      out->nnz += !is_zero_bits(a);
      if (pair) out->nnz += !is_zero_bits(b);
      out->stored_weights += pair ? 2 : 1;
      off += diffs[begin + j];
    }
    out->groups.push_back(rg);
    prev_end = end;
  }
  return true;
}

template SemiCounts CountSemi<float>(const float*, int, int);
template SemiCounts CountSemi<int8_t>(const int8_t*, int, int);
template int CountZerosPad4<float>(const float*, int, int, int*);
template int CountZerosPad4<int8_t>(const int8_t*, int, int, int*);
template int PackWeights<float>(const float*, int, int, int, bool, float*, uint32_t*, int32_t*);
template int PackWeights<int8_t>(const int8_t*, int, int, int, bool, int8_t*, uint32_t*, int32_t*);

}  // namespace pl
