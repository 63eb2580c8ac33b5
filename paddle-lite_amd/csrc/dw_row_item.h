// One output row of a narrow plane of the int8 depthwise 3x3 convolution, from input rows that lie in LDS:
// shared by the depthwise kernel for narrow planes (dwconv_kernels.hip) and by the pointwise kernel that runs
// the following depthwise layer on its own output (image_rows_kernels.hip).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "dwconv_kernels.h"
#include "epilogue.h"

namespace pl {
namespace dwrow {

using epilogue::ActivateT;
using epilogue::ActQuantF;

typedef float v4f __attribute__((ext_vector_type(4)));

struct DwRowStage {
  char* lds_in;      // holds the input bytes from `in_base` on, preceded by 16 bytes of slack
  int64_t in_base;   // offset of the first staged byte in the tensor (a multiple of 16)
};

// Output row oy of `plane` (filter rows wrow as packed bytes (w0, w1, w2, 0), scale s, bias b of its channel): per input row the five aligned dwords around the 16 bytes that start at
// column -pad are read from LDS, shifted into place (v_alignbyte_b32), masked outside the row once, and the byte
// windows of the NOUT outputs slid out of them.  int8 outputs are written byte by byte to dst_i8 (LDS), fp32
// outputs stored to p.out directly.  Lanes that are not `live` compute nothing and store nothing.
template <int STRIDE, int NOUT, int OUT, int ACT, int FIXED = 0>
__device__ __forceinline__ void DwRowItemWith(const DwConvParams& p, const DwRowStage& st, uint32_t plane, const uint32_t (&wrow)[3], float s, float b, int oy, bool live, char* dst_i8) {
  // FIXED: planes of FIXED x FIXED with padding 1, known at compile time (masks and row bounds become constants)
  const int h = FIXED ? FIXED : p.h, w = FIXED ? FIXED : p.w, pad = FIXED ? 1 : p.pad;
  const int oh = FIXED ? (FIXED - 1) / STRIDE + 1 : p.oh, ow = FIXED ? (FIXED - 1) / STRIDE + 1 : p.ow;
  // byte b of a window is column b - pad
  uint32_t mask[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    uint32_t m = 0xffffffffu;
    const int below = pad - 4 * k;          // bytes of the dword in front of column 0
    const int inside = pad + w - 4 * k;   // bytes of the dword, from its first, up to the end of the row
    if (below > 0) m &= 0xffffffffu << (8 * below);
    m = inside <= 0 ? 0u : (inside < 4 ? m & (0xffffffffu >> (8 * (4 - inside))) : m);
    mask[k] = m;
  }
  int acc[NOUT];
#pragma unroll
  for (int j = 0; j < NOUT; ++j) acc[j] = 0;
  if (live) {
    const int iy0 = STRIDE * oy - pad;
    const int64_t plane_at = (int64_t)plane * (uint32_t)(h * w) - st.in_base + 16;  // LDS offset of the plane's first byte
    uint32_t D[3][4];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      // a row outside [0, h) is zero padding: it reads its neighbour and meets a zero filter row below
      const uint32_t at = (uint32_t)(plane_at + (uint32_t)(min(max(iy0 + r, 0), h - 1) * w) - pad);
      const uint32_t* words = reinterpret_cast<const uint32_t*>(st.lds_in + (at & ~3u));
      uint32_t e[5];
#pragma unroll
      for (int k = 0; k < 5; ++k) e[k] = words[k];
#pragma unroll
      for (int k = 0; k < 4; ++k) D[r][k] = __builtin_amdgcn_alignbyte(e[k + 1], e[k], at & 3u);
    }
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const int iy = iy0 + r;
      const int wr = (int)(wrow[r] & ((iy >= 0 && iy < h) ? 0xffffffffu : 0u));
      uint32_t d[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) d[k] = D[r][k] & mask[k];
#pragma unroll
      for (int j = 0; j < NOUT; ++j) {
        const int first = STRIDE * j, k = first / 4, sh = first % 4;
        const int win = sh == 0 ? (int)d[k] : (int)__builtin_amdgcn_alignbyte(k + 1 < 4 ? d[k + 1] : 0u, d[k], sh);
        acc[j] = __builtin_amdgcn_sdot4(win, wr, acc[j], false);
      }
    }
  }
  if (OUT == kOutI8) {
    // the low byte of the truncated value is the int8 output; dst_i8: the item's ow bytes in LDS
    if (live) {
#pragma unroll
      for (int j = 0; j < NOUT; ++j)
        if (j < ow) dst_i8[j] = (char)static_cast<int>(ActQuantF<ACT>(__builtin_fmaf((float)acc[j], s, b), p.act));
    }
  } else if (live) {
    float* dst = static_cast<float*>(p.out) + ((size_t)plane * (uint32_t)oh + (uint32_t)oy) * (uint32_t)ow;
    constexpr int NG = (NOUT + 3) / 4;
#pragma unroll
    for (int q4 = 0; q4 < NG; ++q4) {
      const int n_out = min(4, ow - 4 * q4);
      if (n_out <= 0) break;
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = 4 * q4 + k < NOUT ? ActivateT<ACT>(__builtin_fmaf((float)acc[4 * q4 + k < NOUT ? 4 * q4 + k : 0], s, b), p.act) : 0.0f;
      if (n_out == 4) {  // a four-dword store needs dword alignment only
        *reinterpret_cast<v4f*>(dst + 4 * q4) = v4f{v[0], v[1], v[2], v[3]};
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (k < n_out) dst[4 * q4 + k] = v[k];
      }
    }
  }
}

// The same with the channel's filter rows, scale and bias loaded here (channel c).
template <int STRIDE, int NOUT, int OUT, int ACT>
__device__ __forceinline__ void DwRowItem(const DwConvParams& p, const DwRowStage& st, uint32_t plane, int c, int oy, bool live, char* dst_i8) {
  uint32_t wrow[3] = {0u, 0u, 0u};
  float s = 0.f, b = 0.f;
  if (live) {
    wrow[0] = p.wpack[4 * c];
    wrow[1] = p.wpack[4 * c + 1];
    wrow[2] = p.wpack[4 * c + 2];
    s = p.scale[c];
    b = p.bias[c];
  }
  DwRowItemWith<STRIDE, NOUT, OUT, ACT>(p, st, plane, wrow, s, b, oy, live, dst_i8);
}

}  // namespace dwrow
}  // namespace pl
