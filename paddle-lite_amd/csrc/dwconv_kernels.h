// Device-side interface of the int8 depthwise 3x3 convolution.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "sparse_conv_kernels.h"

namespace pl {

struct DwConvParams {
  const int8_t* x;         // NCHW [batch, channels, h, w]
  void* out;               // NCHW [batch, channels, oh, ow], fp32 or int8
  const uint32_t* wpack;   // [channels][4]: weight rows as bytes (w0, w1, w2, 0); the fourth dword is unused
  const float* scale;      // [channels]
  const float* bias;       // [channels] (zeros when the op has no bias)
  int channels;
  int h, w, oh, ow;
  int pad;                 // 0 or 1, all four sides
  uint32_t planes;         // batch * channels
  int64_t in_bytes;        // planes * h * w
  DevAct act;
  int item_rows;           // output rows per thread: 1, 2 or 4, 0 = chosen by the launcher
  int item_cols;           // groups of 4 output columns per thread: 1, 2 or 4, 0 = chosen by the launcher
  int share_lanes;         // 1: lanes load only their own dwords and exchange the rest; 0: every lane loads all; -1 = chosen by the launcher
  int row_items;           // planes with w + 2 * pad <= 16: 1 = one whole output row per thread, 0 = the item shapes above, -1 = chosen by the launcher
  // filled in by the launcher
  int groups_w;            // column groups per output row
  int items;               // ceil(oh / rows) * groups_w per plane
  int planes_per_group;    // the items of this many planes, laid end to end, fill whole workgroups of 256
  int blocks_per_group;    // planes_per_group * items / 256
  int planes_per_block;    // bound on the planes one workgroup touches
  uint32_t magic_items;    // ceil(2^32 / items) for items >= 2: x / items is mulhi(x, magic) or one less, exactly mulhi for x * items < 2^32
  uint32_t magic_groups;   // likewise for groups_w
  uint32_t magic_blocks;   // likewise for blocks_per_group
  uint32_t magic_channels; // likewise for channels
  int row_lds_in;          // row items: bytes of LDS for the staged input
};

// stride 1 or 2; out_kind kOutF32 or kOutI8.
hipError_t LaunchDwConv3x3(int stride, int out_kind, const DwConvParams& p, hipStream_t stream);

// The int8 -> int8 pointwise layer of image_rows_kernels.hip followed by the int8 -> int8 depthwise layer on its
// output, in one launch: 14 x 14 maps, padding 1, stride 1 or 2.  p.out is not used; d.x is not used (the
// depthwise input never leaves the CU); d.h, d.w, d.oh, d.ow, d.pad, d.channels, d.wpack, d.scale, d.bias, d.act
// and d.out as for LaunchDwConv3x3.
bool ImageRowsDwFits(int M, int K, int hw, int h, int w, int pad, int stride);
hipError_t LaunchImageRowsDw(const ImageMfmaParams& p, const DwConvParams& d, int stride, hipStream_t stream);

}  // namespace pl
