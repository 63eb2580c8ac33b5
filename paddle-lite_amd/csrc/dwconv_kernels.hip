// int8 depthwise 3x3 convolution (one filter per channel), stride 1 or 2,
// zero padding 0 or 1, fused scale / bias / activation and fp32 or int8
// output: the layer that sits between the pointwise convolutions of a
// MobileNet.  Streaming work: every input byte is needed by at most nine
// outputs of its own plane, so there is no staging through LDS; a thread
// makes four neighbouring outputs of one output row from three dword loads
// per input row (the L1 serves the overlap between neighbours), slides byte
// windows out of them with v_alignbyte and multiplies with v_dot4_i32_i8
// against the filter row packed as (w0, w1, w2, 0).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "dwconv_kernels.h"
#include "epilogue.h"

namespace pl {
namespace {

using namespace epilogue;

typedef float v4f __attribute__((ext_vector_type(4)));

// Dword at byte offset `off` of the tensor (any alignment).  SAFE: the
// caller knows all its loads lie inside the tensor.  Otherwise bytes outside
// [0, total) read as zero (only the threads at the two ends of the tensor
// take this path).
template <bool SAFE>
__device__ __forceinline__ uint32_t LoadBytes4(const int8_t* base, int64_t off, int64_t total) {
  if (SAFE) return *reinterpret_cast<const uint32_t*>(base + off);
  uint32_t v = 0;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const int64_t o = off + b;
    if (o >= 0 && o < total) v |= (uint32_t)(uint8_t)base[o] << (8 * b);
  }
  return v;
}

// The four outputs ox0 .. ox0+3 (ox0 = 4g) of output row oy of one plane.
// Window byte i of an input row is column col0 + i with col0 = STRIDE * ox0 -
// pad; output k multiplies window bytes STRIDE*k .. STRIDE*k + 2.  The window
// is cut from the dwords A, B, C that start at columns cb - 4, cb, cb + 4,
// cb = col0 + 1 (for stride 1 and padding 1 that is column 4g: B holds the
// inputs right under the thread's outputs).
template <int STRIDE, int OUT, int ACT, bool SAFE>
__device__ __forceinline__ void DwItem(const DwConvParams& p, uint32_t plane, int c, int oy, int g) {
  const int ox0 = 4 * g;
  const int cb = STRIDE * ox0 - p.pad + 1;  // 0 <= cb < w for every existing output
  const int64_t plane_off = (int64_t)plane * p.h * p.w;
  // Columns outside [0, w) are zero padding (a dword may also run into the
  // next row or plane).  A reaches below column 0 only for g == 0: with
  // padding 1 it is then all padding, without padding its last byte is column 0.
  const uint32_t mA = g == 0 ? (p.pad ? 0u : 0xff000000u) : 0xffffffffu;
  const int in_b = p.w - cb;  // >= 1 bytes of B inside the row
  const uint32_t mB = 0xffffffffu >> (8 * max(4 - in_b, 0));
  const int in_c = in_b - 4;  // bytes of C inside the row (may be <= 0)
  const uint32_t mC = in_c <= 0 ? 0u : 0xffffffffu >> (8 * max(4 - in_c, 0));
  int acc[4] = {0, 0, 0, 0};
#pragma unroll
  for (int r = 0; r < 3; ++r) {
    // a row outside [0, h) is zero padding: its filter row is taken as zero
    const int iy = STRIDE * oy - p.pad + r;
    const bool row_on = iy >= 0 && iy < p.h;
    const int wr = row_on ? (int)p.wpack[4 * c + r] : 0;
    const int64_t row_off = plane_off + (int64_t)min(max(iy, 0), p.h - 1) * p.w;  // a padding row reads its neighbour
    const uint32_t A = LoadBytes4<SAFE>(p.x, row_off + cb - 4, p.in_bytes) & mA;
    const uint32_t B = LoadBytes4<SAFE>(p.x, row_off + cb, p.in_bytes) & mB;
    const uint32_t C = LoadBytes4<SAFE>(p.x, row_off + cb + 4, p.in_bytes) & mC;
    // window bytes 0..3 = columns cb-1 .. cb+2, bytes 4..7 = cb+3 .. cb+6
    const uint32_t win_lo = __builtin_amdgcn_alignbyte(B, A, 3);
    const uint32_t win_hi = __builtin_amdgcn_alignbyte(C, B, 3);
    if (STRIDE == 1) {
      acc[0] = __builtin_amdgcn_sdot4((int)win_lo, wr, acc[0], false);
      acc[1] = __builtin_amdgcn_sdot4((int)__builtin_amdgcn_alignbyte(win_hi, win_lo, 1), wr, acc[1], false);
      acc[2] = __builtin_amdgcn_sdot4((int)__builtin_amdgcn_alignbyte(win_hi, win_lo, 2), wr, acc[2], false);
      acc[3] = __builtin_amdgcn_sdot4((int)__builtin_amdgcn_alignbyte(win_hi, win_lo, 3), wr, acc[3], false);
    } else {
      const uint32_t top = C >> 24;  // window byte 8 = column cb + 7
      acc[0] = __builtin_amdgcn_sdot4((int)win_lo, wr, acc[0], false);
      acc[1] = __builtin_amdgcn_sdot4((int)__builtin_amdgcn_alignbyte(win_hi, win_lo, 2), wr, acc[1], false);
      acc[2] = __builtin_amdgcn_sdot4((int)win_hi, wr, acc[2], false);
      acc[3] = __builtin_amdgcn_sdot4((int)__builtin_amdgcn_alignbyte(top, win_hi, 2), wr, acc[3], false);
    }
  }
  const float s = p.scale[c], b = p.bias[c];
  const int n_out = min(4, p.ow - ox0);
  const size_t o = ((size_t)plane * p.oh + oy) * p.ow + ox0;
  if (OUT == kOutI8) {
    int q[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) q[k] = ActQuantI8<ACT>(__builtin_fmaf((float)acc[k], s, b), p.act);
    int8_t* dst = static_cast<int8_t*>(p.out) + o;
    if (n_out == 4 && (o & 3) == 0) {
      __builtin_nontemporal_store(PackI8x4(q[0], q[1], q[2], q[3]), reinterpret_cast<uint32_t*>(dst));
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (k < n_out) dst[k] = (int8_t)q[k];
    }
  } else {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = ActivateT<ACT>(__builtin_fmaf((float)acc[k], s, b), p.act);
    float* dst = static_cast<float*>(p.out) + o;
    if (n_out == 4 && (o & 3) == 0) {
      __builtin_nontemporal_store(v4f{v[0], v[1], v[2], v[3]}, reinterpret_cast<v4f*>(dst));
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (k < n_out) dst[k] = v[k];
    }
  }
}

template <int STRIDE, int OUT, int ACT>
__device__ __forceinline__ void DwBody(const DwConvParams& p) {
  const uint32_t plane0 = blockIdx.x * (uint32_t)p.planes_per_block;
  const int span = p.planes_per_block * p.items;  // items of this workgroup
  for (int v = threadIdx.x; v < span; v += blockDim.x) {
    const int pl = p.items == 1 ? v : (int)__umulhi((uint32_t)v, p.magic_items);  // v / items
    const int item = v - pl * p.items;
    const uint32_t plane = plane0 + (uint32_t)pl;
    if (plane >= p.planes) break;
    const int oy = p.groups_w == 1 ? item : (int)__umulhi((uint32_t)item, p.magic_groups);  // item / groups_w
    const int g = item - oy * p.groups_w;
    const int c = (int)(plane % (uint32_t)p.channels);
    // every load of the item lies inside the tensor unless the item touches
    // its first or last 8 bytes (dwords A and C reach 4 + 3 bytes past the window)
    const int64_t first = (int64_t)plane * p.h * p.w + (int64_t)max(STRIDE * oy - p.pad, 0) * p.w + (STRIDE * 4 * g - p.pad + 1) - 4;
    const int64_t last = (int64_t)plane * p.h * p.w + (int64_t)min(STRIDE * oy - p.pad + 2, p.h - 1) * p.w + (STRIDE * 4 * g - p.pad + 1) + 8;
    if (first >= 0 && last <= p.in_bytes) {
      DwItem<STRIDE, OUT, ACT, true>(p, plane, c, oy, g);
    } else {
      DwItem<STRIDE, OUT, ACT, false>(p, plane, c, oy, g);
    }
  }
}

template <int STRIDE, int OUT>
__global__ void __launch_bounds__(256) DwConv3x3Kernel(const DwConvParams p) {
  DispatchAct(p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    DwBody<STRIDE, OUT, ACT>(p);
  });
}

// ceil(2^32 / d) for d >= 2 (a divisor of 1 is handled by the kernel: its magic would need 33 bits)
uint32_t Magic(int d) { return d <= 1 ? 0u : (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d); }

}  // namespace

hipError_t LaunchDwConv3x3(int stride, int out_kind, const DwConvParams& p, hipStream_t stream) {
  if (p.planes == 0 || p.oh <= 0 || p.ow <= 0) return hipSuccess;
  if ((stride != 1 && stride != 2) || (p.pad != 0 && p.pad != 1) || (out_kind != kOutF32 && out_kind != kOutI8)) return hipErrorInvalidValue;
  DwConvParams q = p;
  q.groups_w = (p.ow + 3) / 4;
  const int64_t items = (int64_t)p.oh * q.groups_w;
  // the magic divisions need v * items < 2^32 for every v below the workgroup's span
  if (items > 46000) return hipErrorInvalidValue;
  q.items = (int)items;
  q.planes_per_block = q.items >= 256 ? 1 : 256 / q.items;
  q.magic_items = Magic(q.items);
  q.magic_groups = Magic(q.groups_w);
  const uint32_t blocks = (p.planes + q.planes_per_block - 1) / q.planes_per_block;
  dim3 grid(blocks), block(256);
  if (stride == 1) {
    if (out_kind == kOutI8) {
      hipLaunchKernelGGL((DwConv3x3Kernel<1, kOutI8>), grid, block, 0, stream, q);
    } else {
      hipLaunchKernelGGL((DwConv3x3Kernel<1, kOutF32>), grid, block, 0, stream, q);
    }
  } else {
    if (out_kind == kOutI8) {
      hipLaunchKernelGGL((DwConv3x3Kernel<2, kOutI8>), grid, block, 0, stream, q);
    } else {
      hipLaunchKernelGGL((DwConv3x3Kernel<2, kOutF32>), grid, block, 0, stream, q);
    }
  }
  return hipGetLastError();
}

}  // namespace pl
