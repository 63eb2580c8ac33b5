// Host-side handling of the sparse_conv2d weight layout
// (NonZeroWeights / OcNonZeros / Diffs): the opt-time packers and the
// run-time decoder that turns byte offsets back into channel indices.
// Pure C++, no device code.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace pl {

enum class WeightType : int { kFloat = 0, kInt8 = 1 };

// Result of the block-density analysis the detect pass runs on a dense
// [oc x ic] weight matrix.
// reference: lite/core/optimizer/mir/sparse_conv_detect_pass.cc:303-368
struct SemiCounts {
  int zeros = 0;            // oc*ic - count_nonzeroes (what the pass thresholds)
  int count_nonzeroes = 0;  // weights the chosen layout stores
  int count_channels = 0;
  int count_blocks = 0;     // index entries the chosen layout stores
  int flag_semi = 0;
};

template <typename T>
SemiCounts CountSemi(const T* dense, int oc, int ic);

// reference: sparse_conv_detect_pass.cc:480-517
template <typename T>
int CountZerosPad4(const T* dense, int oc, int ic, int* num_build_nonzeroes);

// The three packers behind one call, chosen like the pass does
// (sparse_conv_detect_pass.cc:732-780). Returns first_ic.
// reference: sparse_conv_detect_pass.cc:35-91 (unpadded), :93-194 (padded),
//            :196-301 (semi)
template <typename T>
int PackWeights(const T* dense, int oc, int ic, int im_size, bool semi,
                T* nonzero_weights, uint32_t* oc_nonzeros, int32_t* diffs);

// One output row (or a pair of rows sharing indices) with absolute input
// channel indices.
struct RowGroup {
  int row0 = 0;
  int nrows = 1;          // 1 or 2
  uint32_t first = 0;     // first entry in DecodedLayout::ic / weight bits
  uint32_t count = 0;
};

struct DecodedLayout {
  int oc = 0, ic = 0;
  bool semi = false;
  WeightType type = WeightType::kFloat;
  std::vector<RowGroup> groups;
  std::vector<uint32_t> ic_index;   // per entry
  // per entry: 1 (unstructured) or 2 (semi) weights, as raw 32-bit patterns
  // (float bits, or the int8 value sign-extended)
  std::vector<uint32_t> w0, w1;
  int64_t nnz = 0;             // nonzero weights
  int64_t stored_weights = 0;  // weights present in the layout
};

// Walks OcNonZeros / Diffs with the per-row start rules of the math
// functions (lite/backends/arm/math/sparse_conv_impl.cc:1226-1243,
// :2464-2475; sparse_semi_conv_impl.cc:1788-1823) and checks every index.
// Returns false and fills *error when the arrays do not describe a matrix.
bool DecodeLayout(WeightType type, bool semi, const void* nonzero_weights,
                  int64_t n_weights, const uint32_t* oc_nonzeros,
                  const int32_t* diffs, int64_t n_diffs, int first_ic, int oc,
                  int ic, int im_size, DecodedLayout* out, std::string* error);

}  // namespace pl
