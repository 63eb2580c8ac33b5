// Thin C entry points around the reference's own weight packers as its math
// tests carry them (lite/tests/math/conv_ut.h:183-538: ComputeSparseZeros,
// ComputeSemiSparseZeros, ComputeSparseWeight x2, ComputeSemiSparseWeight;
// the same algorithms as the members of SparseConvDetectPass,
// lite/core/optimizer/mir/sparse_conv_detect_pass.cc:35-517).  The header as a
// whole needs gflags and the x86 conv kernel's dependencies, so the Makefile
// takes exactly those lines of it into oracle/_ref/conv_ut_packers.inc at
// build time (a build product beside the .so, never committed) and this file
// compiles them against the reference's real Tensor classes.
// TEST INFRASTRUCTURE ONLY: pins the oracle's and the library's packers.
#include <cstdint>
#include <cstring>
#include <vector>

#include "lite/core/tensor.h"

typedef paddle::lite::DDim DDim;
typedef paddle::lite::Tensor Tensor;

#include "conv_ut_packers.inc"

namespace {
template <typename T>
void Fill(Tensor* t, const void* src, int rows, int cols) {
  t->Resize(DDim(std::vector<int64_t>{rows, cols}));
  std::memcpy(t->mutable_data<T>(), src, sizeof(T) * rows * cols);
}

template <typename T>
int Pack(int layout, const void* w, int M, int K, int N, void* nonzero, int64_t n_w, uint32_t* oc_nonzeros, int32_t* diffs, int64_t n_d) {
  Tensor wt, nz, oc, df;
  Fill<T>(&wt, w, M, K);
  nz.Resize(DDim(std::vector<int64_t>{n_w > 0 ? n_w : 1}));
  oc.Resize(DDim(std::vector<int64_t>{M}));
  df.Resize(DDim(std::vector<int64_t>{n_d > 0 ? n_d : 1}));
  nz.mutable_data<T>();
  // the semi packer writes one count per row pair and leaves the rest of the M entries alone
  std::memset(oc.mutable_data<uint32_t>(), 0, sizeof(uint32_t) * M);
  df.mutable_data<int32_t>();
  int first_ic = 0;
  if (layout == 0) {  // unpadded rows (the int8 choice of the pass)
    int nb = 0;
    const int zeros = ComputeSparseZeros<T>(&wt, &nb, M, K);
    first_ic = ComputeSparseWeight<T>(&wt, M, K, N, M * K - zeros, &nz, &oc, &df);
  } else if (layout == 1) {  // rows padded to four (the fp32 choice)
    int nb = 0;
    const int zeros = ComputeSparseZeros<T>(&wt, &nb, M, K);
    first_ic = ComputeSparseWeight<T>(&wt, M, K, N, M * K - zeros, nb, &nz, &oc, &df);
  } else {  // semi-structured
    int cn = 0, cc = 0, cb = 0, fs = 0;
    ComputeSemiSparseZeros<T>(&wt, &cn, &cc, &cb, &fs, M, K);
    // the counts describe the semi layout only when the pass's block rule fires, which is when the
    // reference calls this packer (lite/core/optimizer/mir/sparse_conv_detect_pass.cc:732-760)
    if (!fs || cn != n_w || cb != n_d) return -1;
    first_ic = ComputeSemiSparseWeight<T>(&wt, M, K, N, cn, cc, cb, &nz, &oc, &df);
  }
  std::memcpy(nonzero, nz.data<T>(), sizeof(T) * n_w);
  std::memcpy(oc_nonzeros, oc.data<uint32_t>(), sizeof(uint32_t) * M);
  std::memcpy(diffs, df.data<int32_t>(), sizeof(int32_t) * n_d);
  return first_ic;
}
}  // namespace

extern "C" {

// dtype: 0 fp32, 1 int8.  Returns the zero count; *num_build = elements of the padded layout.
int ref_count_zeros_pad4(int dtype, const void* w, int rows, int cols, int* num_build) {
  Tensor t;
  if (dtype == 0) {
    Fill<float>(&t, w, rows, cols);
    return ComputeSparseZeros<float>(&t, num_build, rows, cols);
  }
  Fill<int8_t>(&t, w, rows, cols);
  return ComputeSparseZeros<int8_t>(&t, num_build, rows, cols);
}

int ref_count_semi(int dtype, const void* w, int rows, int cols, int* count_nonzeroes, int* count_channels, int* count_blocks, int* flag_semi) {
  Tensor t;
  if (dtype == 0) {
    Fill<float>(&t, w, rows, cols);
    return ComputeSemiSparseZeros<float>(&t, count_nonzeroes, count_channels, count_blocks, flag_semi, rows, cols);
  }
  Fill<int8_t>(&t, w, rows, cols);
  return ComputeSemiSparseZeros<int8_t>(&t, count_nonzeroes, count_channels, count_blocks, flag_semi, rows, cols);
}

// layout: 0 unpadded, 1 padded to four, 2 semi.  The caller sizes the outputs
// (n_w weights, M counts, n_d offsets).  Returns first_ic.
int ref_pack(int dtype, int layout, const void* w, int M, int K, int N, void* nonzero, int64_t n_w, uint32_t* oc_nonzeros, int32_t* diffs, int64_t n_d) {
  return dtype == 0 ? Pack<float>(layout, w, M, K, N, nonzero, n_w, oc_nonzeros, diffs, n_d) : Pack<int8_t>(layout, w, M, K, N, nonzero, n_w, oc_nonzeros, diffs, n_d);
}

}  // extern "C"
