// int8 depthwise 3x3 convolution (one filter per channel), stride 1 or 2,
// zero padding 0 or 1, fused scale / bias / activation and fp32 or int8
// output: the layer that sits between the pointwise convolutions of a
// MobileNet.  Streaming work: every input byte is needed by at most nine
// outputs of its own plane, so there is no staging through LDS; a thread
// makes four neighbouring outputs of several output rows from three dword loads
// per input row (the L1 serves the overlap between neighbours), slides byte
// windows out of them with v_alignbyte and multiplies with v_dot4_i32_i8
// against the filter row packed as (w0, w1, w2, 0).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "dw_row_item.h"
#include "dwconv_kernels.h"
#include "epilogue.h"
#include "launch_lds.h"

namespace pl {
namespace {

using namespace epilogue;

typedef float v4f __attribute__((ext_vector_type(4)));

// Dword at `ptr` (any alignment).  SAFE: the caller knows that the four
// bytes lie inside the tensor.  Otherwise bytes outside [lo, hi) read as zero
// (only the workgroups at the two ends of the tensor take this path, but the
// kernel lasts as long as they do): the load is moved inside the tensor and
// the value shifted, without a branch, so that all loads of an item are in
// flight together as on the safe path.
template <bool SAFE>
__device__ __forceinline__ uint32_t LoadBytes4(const int8_t* ptr, const int8_t* lo, const int8_t* hi) {
  if (SAFE) return *reinterpret_cast<const uint32_t*>(ptr);
  if (hi - lo < 4) {
    uint32_t v = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b)
      if (ptr + b >= lo && ptr + b < hi) v |= (uint32_t)(uint8_t)ptr[b] << (8 * b);
    return v;
  }
  const int8_t* at = ptr < lo ? lo : (ptr > hi - 4 ? hi - 4 : ptr);
  const uint32_t v = *reinterpret_cast<const uint32_t*>(at);
  const int d = (int)(ptr - at);  // < 0: the dword starts below the tensor, > 0: it ends above
  const uint32_t up = d > -4 ? v << (8 * (-d & 3)) : 0u;
  const uint32_t down = d < 4 ? v >> (8 * (d & 3)) : 0u;
  return d == 0 ? v : (d < 0 ? up : down);
}

// One item: 4 * CG neighbouring outputs (from column ox0 = 4 * CG * g) of the
// R output rows R*oyr .. R*oyr + R-1 of one plane.  With col0 = STRIDE * ox0 -
// pad the column of the first input under the first output, the item reads,
// per input row, the K dwords that start at columns cb - 4, cb, cb + 4, ...
// (cb = col0 + 1; for stride 1 and padding 1 that is column ox0 itself).
// Output j multiplies the three bytes from column col0 + STRIDE * j on: they
// are the low bytes of the dword pair (k, k + 1) shifted right by sh bytes,
// k = (STRIDE*j + 3) / 4, sh = (STRIDE*j + 3) % 4, both compile-time values.
// Neighbouring output rows share 2 of their 3 input rows at stride 1 (1 of 3
// at stride 2).
template <int STRIDE, int R, int CG, int OUT, int ACT, bool SAFE>
__device__ __forceinline__ void DwItem(const DwConvParams& p, uint32_t plane, int c, int oyr, int g) {
  constexpr int kRows = 3 + STRIDE * (R - 1);                  // input rows under R output rows
  constexpr int NOUT = 4 * CG;                                 // outputs per row
  constexpr int K = (STRIDE * (NOUT - 1) + 3 + 2) / 4 + 1;     // dwords per input row (the last window starts in dword K - 2)
  const int ox0 = NOUT * g;
  const int cb = STRIDE * ox0 - p.pad + 1;  // 0 <= cb < w for every existing output
  const int8_t* plane_ptr = p.x + (int64_t)plane * (uint32_t)(p.h * p.w);
  // Columns outside [0, w) are zero padding (a dword may also run into the
  // next row or plane).  Only dword 0 can reach below column 0, and only for
  // g == 0: with padding 1 it is then all padding, without padding its last
  // byte is column 0.
  uint32_t mask[K];
  mask[0] = g == 0 ? (p.pad ? 0u : 0xff000000u) : 0xffffffffu;
#pragma unroll
  for (int k = 1; k < K; ++k) {
    const int inside = p.w - (cb + 4 * (k - 1));  // bytes of dword k inside the row, from its first byte
    mask[k] = inside <= 0 ? 0u : 0xffffffffu >> (8 * max(4 - inside, 0));
  }
  const uint32_t wrow[3] = {p.wpack[4 * c], p.wpack[4 * c + 1], p.wpack[4 * c + 2]};
  const int iy0 = STRIDE * R * oyr - p.pad;
  int acc[R][NOUT];
#pragma unroll
  for (int o = 0; o < R; ++o)
#pragma unroll
    for (int j = 0; j < NOUT; ++j) acc[o][j] = 0;
  uint32_t D[kRows][K];
  const int8_t* rows[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    // a row outside [0, h) is zero padding: it reads its neighbour and meets a zero filter row below
    rows[r] = plane_ptr + (uint32_t)(min(max(iy0 + r, 0), p.h - 1) * p.w) + cb;
  }
  if (CG == 1 && p.share_lanes) {
    // Neighbouring lanes hold neighbouring column groups of the same rows, and
    // the dwords a lane needs beside its own STRIDE dwords are its
    // neighbours' own: each lane loads only its own bytes (the wavefront's
    // loads are then contiguous and disjoint) and takes dword 0 from the lane
    // below and, at stride 1, dword 2 from the lane above, with wavefront
    // shifts.  Lanes at the end of a row or of the wavefront load them instead.
    constexpr int OWN = STRIDE;  // dwords 1 .. OWN are the lane's own
    const int lane = (int)(threadIdx.x & 63);
    const bool below_ok = g > 0 && lane > 0;
    const bool above_ok = g + 1 < p.groups_w && lane < 63;
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int k = 1; k <= OWN; ++k) D[r][k] = LoadBytes4<SAFE>(rows[r] + 4 * (k - 1), p.x, p.x + p.in_bytes);
    uint32_t edge_lo[kRows], edge_hi[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) edge_lo[r] = edge_hi[r] = 0u;
    if (!below_ok && mask[0] != 0u) {
#pragma unroll
      for (int r = 0; r < kRows; ++r) edge_lo[r] = LoadBytes4<SAFE>(rows[r] - 4, p.x, p.x + p.in_bytes);
    }
    if (STRIDE == 1 && !above_ok && mask[2] != 0u) {
#pragma unroll
      for (int r = 0; r < kRows; ++r) edge_hi[r] = LoadBytes4<SAFE>(rows[r] + 4, p.x, p.x + p.in_bytes);
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      // wave_shr:1 (0x138): lane i takes lane i - 1's value; wave_shl:1 (0x130): lane i + 1's
      const uint32_t from_below = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)D[r][OWN], 0x138, 0xf, 0xf, false);
      D[r][0] = below_ok ? from_below : edge_lo[r];
      if (STRIDE == 1) {
        const uint32_t from_above = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)D[r][1], 0x130, 0xf, 0xf, false);
        D[r][2] = above_ok ? from_above : edge_hi[r];
      }
    }
  } else {
    // every lane loads all its dwords (the compiler merges them into one
    // load per row; the L1 serves the overlap between neighbouring lanes)
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int k = 0; k < K; ++k) D[r][k] = LoadBytes4<SAFE>(rows[r] + 4 * (k - 1), p.x, p.x + p.in_bytes);
  }
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int iy = iy0 + r;
    const uint32_t row_on = (iy >= 0 && iy < p.h) ? 0xffffffffu : 0u;
    uint32_t d[K];
#pragma unroll
    for (int k = 0; k < K; ++k) d[k] = D[r][k] & mask[k];
    int win[NOUT];
#pragma unroll
    for (int j = 0; j < NOUT; ++j) {
      const int first = STRIDE * j + 3;  // byte index of the window's first byte in the dword sequence
      const int k = first / 4, sh = first % 4;
      win[j] = sh == 0 ? (int)d[k] : (int)__builtin_amdgcn_alignbyte(k + 1 < K ? d[k + 1] : 0u, d[k], sh);
    }
#pragma unroll
    for (int o = 0; o < R; ++o) {
      const int fr = r - STRIDE * o;  // filter row this input row meets in output row o
      if (fr < 0 || fr > 2) continue;
      const int wr = (int)(wrow[fr] & row_on);
#pragma unroll
      for (int j = 0; j < NOUT; ++j) acc[o][j] = __builtin_amdgcn_sdot4(win[j], wr, acc[o][j], false);
    }
  }
  const float s = p.scale[c], b = p.bias[c];
#pragma unroll
  for (int o = 0; o < R; ++o) {
    const int oy = R * oyr + o;
    if (oy >= p.oh) break;
    const size_t row_at = ((size_t)plane * (uint32_t)p.oh + (uint32_t)oy) * (uint32_t)p.ow + (uint32_t)ox0;
    if (OUT == kOutI8) {
      uint32_t packed[CG];
#pragma unroll
      for (int q4 = 0; q4 < CG; ++q4) {
        float q[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) q[k] = ActQuantF<ACT>(__builtin_fmaf((float)acc[o][4 * q4 + k], s, b), p.act);
        packed[q4] = TruncPackI8x4(q[0], q[1], q[2], q[3]);
      }
      int8_t* dst = static_cast<int8_t*>(p.out) + row_at;
      // global memory takes dword and short stores at any byte address
      if (CG > 1 && ox0 + 4 * CG <= p.ow) {
        // the whole item in one store: the wavefront's stores are then contiguous
        if (CG == 2) {
          *reinterpret_cast<uint2*>(dst) = make_uint2(packed[0], packed[CG - 1]);
        } else {
          *reinterpret_cast<uint4*>(dst) = make_uint4(packed[0], packed[1 % CG], packed[2 % CG], packed[3 % CG]);
        }
      } else {
#pragma unroll
        for (int q4 = 0; q4 < CG; ++q4) {
          const int n_out = min(4, p.ow - (ox0 + 4 * q4));
          if (n_out <= 0) break;
          if (n_out == 4) {
            *reinterpret_cast<uint32_t*>(dst + 4 * q4) = packed[q4];
          } else {
            if (n_out >= 2) *reinterpret_cast<uint16_t*>(dst + 4 * q4) = (uint16_t)packed[q4];
            if (n_out == 1) dst[4 * q4] = (int8_t)packed[q4];
            if (n_out == 3) dst[4 * q4 + 2] = (int8_t)(packed[q4] >> 16);
          }
        }
      }
    } else {
#pragma unroll
      for (int q4 = 0; q4 < CG; ++q4) {
        const int n_out = min(4, p.ow - (ox0 + 4 * q4));
        if (n_out <= 0) break;
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = ActivateT<ACT>(__builtin_fmaf((float)acc[o][4 * q4 + k], s, b), p.act);
        float* dst = static_cast<float*>(p.out) + row_at + 4 * q4;
        if (n_out == 4) {  // a four-dword store needs dword alignment only
          *reinterpret_cast<v4f*>(dst) = v4f{v[0], v[1], v[2], v[3]};
        } else {
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (k < n_out) dst[k] = v[k];
        }
      }
    }
  }
}

// x / d for any 32-bit x with magic = ceil(2^32 / d), d >= 2: the multiply-high
// is the quotient or one more.
__device__ __forceinline__ uint32_t DivMagic(uint32_t x, uint32_t d, uint32_t magic) {
  if (d == 1) return x;
  const uint32_t q = __umulhi(x, magic);
  return q * d > x ? q - 1 : q;
}

// One item per thread and no loop: a wavefront that has stores in flight can
// wait for later loads only by waiting for the stores as well, so a second
// item in the same thread would start after the first one's stores have
// reached memory.
template <int STRIDE, int R, int CG, int OUT, int ACT, bool SAFE>
__device__ __forceinline__ void DwItems(const DwConvParams& p, uint32_t plane0, int v) {
  // v = item of plane0 + thread index, below items + 256: v / items is 0 or 1
  // for planes of 256 items and more, else v * items < 2^32 and the
  // multiply-high is exact
  const int pl = p.items >= 256 ? (v >= p.items ? 1 : 0) : (p.items == 1 ? v : (int)__umulhi((uint32_t)v, p.magic_items));
  const int item = v - pl * p.items;
  const uint32_t plane = plane0 + (uint32_t)pl;
  if (plane >= p.planes) return;
  const int oyr = (int)DivMagic((uint32_t)item, (uint32_t)p.groups_w, p.magic_groups);  // item / groups_w
  const int g = item - oyr * p.groups_w;
  int c = (int)(plane0 - DivMagic(plane0, (uint32_t)p.channels, p.magic_channels) * (uint32_t)p.channels) + pl;  // plane0 % channels (uniform) + pl
  if (c >= p.channels) c = p.channels > p.planes_per_block ? c - p.channels : c % p.channels;
  DwItem<STRIDE, R, CG, OUT, ACT, SAFE>(p, plane, c, oyr, g);
}

template <int STRIDE, int R, int CG, int OUT, int ACT>
__device__ __forceinline__ void DwBody(const DwConvParams& p) {
  // The items of planes_per_group planes are laid end to end and cut into
  // pieces of 256, one per workgroup; planes_per_group * items is a multiple
  // of 256, so every lane of every workgroup has an item (but for the planes
  // past the end of the tensor in the last group).
  const uint32_t group = DivMagic(blockIdx.x, (uint32_t)p.blocks_per_group, p.magic_blocks);
  const uint32_t first = 256u * (blockIdx.x - group * (uint32_t)p.blocks_per_group);  // first item of the workgroup within its group
  const uint32_t pl0 = DivMagic(first, (uint32_t)p.items, p.magic_items);
  const uint32_t plane0 = group * (uint32_t)p.planes_per_group + pl0;
  const int v = (int)(first - pl0 * (uint32_t)p.items) + (int)threadIdx.x;
  // The dwords of a row reach 4 bytes before its first column and up to 15
  // bytes past its last one: only the workgroups with the first and the last
  // plane can leave the tensor (with planes of at least 16 bytes, so that one
  // neighbouring plane covers the reach)
  if (plane0 > 0 && plane0 + (uint32_t)p.planes_per_block < p.planes && p.h * p.w >= 16) {
    DwItems<STRIDE, R, CG, OUT, ACT, true>(p, plane0, v);
  } else {
    DwItems<STRIDE, R, CG, OUT, ACT, false>(p, plane0, v);
  }
}

// R output rows by 4 * CG columns per item (the per-item address and mask
// arithmetic is shared by all of them).
template <int STRIDE, int R, int CG, int OUT>
__global__ void __launch_bounds__(256) DwConv3x3Kernel(const DwConvParams p) {
  DispatchAct(p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    DwBody<STRIDE, R, CG, OUT, ACT>(p);
  });
}

// ---------------------------------------------------------------------------
// Narrow planes (w + 2 * pad <= 16: the 14 x 14 and 7 x 7 maps).  Their rows
// start at any byte address, and global memory is slow with that: the general
// kernel spends 8.5 us on 64 x 512 planes of 14 x 14 whatever its instruction
// count.  Here an item is one whole output row of a plane (up to 14 outputs at
// stride 1, 7 at stride 2), items are numbered through all planes, 256 per
// workgroup, one per thread, and global memory is touched in aligned 16-byte
// pieces only:
//   * the input bytes the workgroup's rows need are one contiguous range; it
//     is copied to LDS as whole 16-byte pieces (tensors are 16-byte aligned);
//   * per input row a thread reads the five aligned dwords around the 16 bytes
//     that start at column -pad from LDS, shifts them into place
//     (v_alignbyte_b32), masks the bytes outside the row once and slides the
//     byte windows of its outputs out of them;
//   * int8 outputs go to LDS byte by byte (the workgroup's output rows are
//     one contiguous range too) and leave as aligned 16-byte pieces; fp32
//     outputs are stored directly (dword aligned).
using dwrow::DwRowItem;
using dwrow::DwRowStage;

template <int STRIDE, int NOUT, int OUT>
__global__ void __launch_bounds__(256) DwRowKernel(const DwConvParams p) {
  extern __shared__ uint4 dw_lds[];
  const int tid = (int)threadIdx.x;
  const uint32_t total = p.planes * (uint32_t)p.oh;  // items
  const uint32_t first = 256u * blockIdx.x, last = min(first + 255u, total - 1u);
  const uint32_t plane_a = DivMagic(first, (uint32_t)p.oh, p.magic_items), plane_b = DivMagic(last, (uint32_t)p.oh, p.magic_items);
  const int oy_a = (int)(first - plane_a * (uint32_t)p.oh), oy_b = (int)(last - plane_b * (uint32_t)p.oh);
  const int64_t hw = (int64_t)p.h * p.w;
  // the input bytes the workgroup's rows need, widened to whole 16-byte pieces
  const int64_t need_lo = (int64_t)plane_a * hw + (int64_t)max(0, STRIDE * oy_a - p.pad) * p.w;
  const int64_t need_hi = (int64_t)plane_b * hw + (int64_t)min(p.h, STRIDE * oy_b - p.pad + 3) * p.w;
  DwRowStage st;
  st.in_base = need_lo & ~(int64_t)15;
  st.lds_in = reinterpret_cast<char*>(dw_lds);
  char* lds_out = st.lds_in + p.row_lds_in;  // int8 output rows of the workgroup, item-major
  const int pieces = (int)((need_hi - st.in_base + 15) >> 4);
  uint4 piece[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int j = tid + 256 * u;
    const int64_t at = st.in_base + 16 * (int64_t)j;
    piece[u] = make_uint4(0, 0, 0, 0);
    if (j < pieces) {
      if (at + 16 <= p.in_bytes) {
        piece[u] = *reinterpret_cast<const uint4*>(p.x + at);
      } else {  // the tensor's last, partial piece
        uint32_t w4[4] = {0, 0, 0, 0};
        for (int t = 0; t < 16; ++t)
          if (at + t < p.in_bytes) w4[t >> 2] |= (uint32_t)(uint8_t)p.x[at + t] << (8 * (t & 3));
        piece[u] = make_uint4(w4[0], w4[1], w4[2], w4[3]);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int j = tid + 256 * u;
    if (j < pieces) *reinterpret_cast<uint4*>(st.lds_in + 16 + 16 * j) = piece[u];
  }
  __syncthreads();
  const uint32_t item = first + (uint32_t)tid;
  const bool live = item < total;
  const uint32_t plane = live ? DivMagic(item, (uint32_t)p.oh, p.magic_items) : plane_b;
  const int oy = live ? (int)(item - plane * (uint32_t)p.oh) : oy_b;
  const int c = (int)(plane - DivMagic(plane, (uint32_t)p.channels, p.magic_channels) * (uint32_t)p.channels);
  DispatchAct(p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    DwRowItem<STRIDE, NOUT, OUT, ACT>(p, st, plane, c, oy, live, lds_out + (uint32_t)tid * (uint32_t)p.ow);
  });
  if (OUT == kOutI8) {
    __syncthreads();
    // the workgroup's output rows: 256 * ow bytes from item `first` on, a multiple of 16 at a multiple of 16
    const int64_t out_at = (int64_t)first * p.ow + 16 * (int64_t)tid;
    const int64_t out_end = (int64_t)total * p.ow;
    if (tid < 16 * p.ow) {
      int8_t* dst = static_cast<int8_t*>(p.out) + out_at;
      const uint4 v = *reinterpret_cast<const uint4*>(lds_out + 16 * tid);
      if (out_at + 16 <= out_end) {
        *reinterpret_cast<uint4*>(dst) = v;
      } else {  // the tensor's last, partial piece
        const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
        for (int t = 0; t < 16; ++t)
          if (out_at + t < out_end) dst[t] = (int8_t)(w4[t >> 2] >> (8 * (t & 3)));
      }
    }
  }
}

template <int STRIDE, int NOUT>
hipError_t LaunchRows(int out_kind, dim3 grid, size_t lds, hipStream_t stream, const DwConvParams& q) {
  if (out_kind == kOutI8) return LaunchWithLds(DwRowKernel<STRIDE, NOUT, kOutI8>, grid, dim3(256), lds, stream, q);
  return LaunchWithLds(DwRowKernel<STRIDE, NOUT, kOutF32>, grid, dim3(256), lds, stream, q);
}

template <int STRIDE, int R, int CG>
void LaunchShape(int out_kind, dim3 grid, hipStream_t stream, const DwConvParams& q) {
  if (out_kind == kOutI8) {
    hipLaunchKernelGGL((DwConv3x3Kernel<STRIDE, R, CG, kOutI8>), grid, dim3(256), 0, stream, q);
  } else {
    hipLaunchKernelGGL((DwConv3x3Kernel<STRIDE, R, CG, kOutF32>), grid, dim3(256), 0, stream, q);
  }
}

// ceil(2^32 / d) for d >= 2 (a divisor of 1 is handled by the kernel: its magic would need 33 bits)
uint32_t Magic(int d) { return d <= 1 ? 0u : (uint32_t)(((1ull << 32) + (uint64_t)d - 1) / (uint64_t)d); }

}  // namespace

hipError_t LaunchDwConv3x3(int stride, int out_kind, const DwConvParams& p, hipStream_t stream) {
  if (p.planes == 0 || p.oh <= 0 || p.ow <= 0) return hipSuccess;
  if ((stride != 1 && stride != 2) || (p.pad != 0 && p.pad != 1) || (out_kind != kOutF32 && out_kind != kOutI8)) return hipErrorInvalidValue;
  DwConvParams q = p;
  // Item shape: output rows by groups of four output columns per thread.
  // More outputs per thread lower the instruction count per output, fewer
  // leave more wavefronts to hide the load latency.  Measured on the MobileNet
  // shapes at batch 64 (kernel us for rows x groups 2x1 / 4x1 / 1x2 / 2x2 /
  // 1x4): stride 1: 112x112 28.0 / - / - / 19.7 / 20.1, 56x56 26.5 / 24.4 /
  // - / 19.4 / 22.6, 28x28 14.2 / 14.1 / - / 12.9 / 13.3, 14x14 9.7 / 9.8 /
  // - / 9.8 / -; stride 2 (output size): 56x56 20.5 / - / 16.4 / 19.9 / 21.3,
  // 28x28 11.2 / - / 10.2 / 11.8 / 12.0.
  int rows = p.item_rows, cg = p.item_cols;
  const bool rows_given = rows == 1 || rows == 2 || rows == 4, cols_given = cg == 1 || cg == 2 || cg == 4;
  // Narrow planes of 16-byte aligned tensors: one output row per thread, global memory touched in aligned
  // 16-byte pieces only, unless an item shape is asked for.  The input range of a workgroup (the planes
  // its 256 rows touch) must fit 16 KB of LDS.
  {
    const int64_t planes_per_wg = (256 + p.oh - 1) / p.oh + 1;
    const int64_t lds_in = ((planes_per_wg * p.h * p.w + 15) / 16 + 6) * 16;  // 16 bytes in front, alignment of the first piece, windows that reach past the last row
    const bool aligned = reinterpret_cast<uintptr_t>(p.x) % 16 == 0 && reinterpret_cast<uintptr_t>(p.out) % 16 == 0;
    if (p.w + 2 * p.pad <= 16 && lds_in <= 16384 && aligned && (p.row_items > 0 || (p.row_items < 0 && !rows_given && !cols_given))) {
      const uint64_t items64 = (uint64_t)p.planes * (uint64_t)p.oh;
      if (items64 >= (1ull << 31)) return hipErrorInvalidValue;
      q.magic_items = Magic(p.oh);
      q.magic_channels = Magic(p.channels);
      q.row_lds_in = (int)lds_in;
      const size_t lds = (size_t)lds_in + (out_kind == kOutI8 ? (size_t)256 * p.ow : 0);
      dim3 row_grid((uint32_t)((items64 + 255) / 256));
      if (stride == 1) return p.ow <= 7 ? LaunchRows<1, 7>(out_kind, row_grid, lds, stream, q) : LaunchRows<1, 14>(out_kind, row_grid, lds, stream, q);
      return LaunchRows<2, 7>(out_kind, row_grid, lds, stream, q);
    }
  }
  if (!cols_given) cg = stride == 1 ? ((p.oh >= 24 && p.ow >= 24) ? 2 : 1) : (p.ow >= 14 ? 2 : 1);
  if (!rows_given) rows = stride == 1 ? 2 : (cg == 2 ? 1 : 2);
  if (stride == 2 && rows == 4) rows = 2;
  if (rows * cg > 8 || (rows == 1 && cg == 1)) return hipErrorInvalidValue;  // 8 to 32 outputs per thread
  // Rows that are not 4-byte aligned make the overlapping per-lane loads
  // slow; there the lanes share their dwords instead (measured: 14x14 planes
  // 12.7 -> 10.4 us, 112x112 planes 28.3 -> 31.5 us with sharing).
  q.share_lanes = cg != 1 ? 0 : (p.share_lanes >= 0 ? p.share_lanes : (p.w % 4 != 0 ? 1 : 0));
  q.groups_w = (p.ow + 4 * cg - 1) / (4 * cg);
  const int64_t items = (int64_t)((p.oh + rows - 1) / rows) * q.groups_w;
  // 256 * items (the span of a group of planes) must fit 32 bits
  if (items >= (1 << 24)) return hipErrorInvalidValue;
  q.items = (int)items;
  // planes per group: the smallest count whose items fill whole workgroups
  int gcd = 256;
  for (int a = q.items % 256; a != 0;) {
    const int t = gcd % a;
    gcd = a;
    a = t;
  }
  q.planes_per_group = 256 / gcd;
  q.blocks_per_group = (int)((int64_t)q.planes_per_group * q.items / 256);
  q.planes_per_block = 256 / q.items + 2;  // bound on the planes one workgroup touches
  q.magic_items = Magic(q.items);
  q.magic_groups = Magic(q.groups_w);
  q.magic_blocks = Magic(q.blocks_per_group);
  q.magic_channels = Magic(p.channels);
  const uint64_t blocks64 = (uint64_t)((p.planes + q.planes_per_group - 1) / q.planes_per_group) * (uint64_t)q.blocks_per_group;
  if (blocks64 >= (1ull << 31)) return hipErrorInvalidValue;
  const uint32_t blocks = (uint32_t)blocks64;
  dim3 grid(blocks);
  const int shape = 100 * stride + 10 * rows + cg;
  switch (shape) {
    case 121:
      LaunchShape<1, 2, 1>(out_kind, grid, stream, q);
      break;
    case 141:
      LaunchShape<1, 4, 1>(out_kind, grid, stream, q);
      break;
    case 112:
      LaunchShape<1, 1, 2>(out_kind, grid, stream, q);
      break;
    case 122:
      LaunchShape<1, 2, 2>(out_kind, grid, stream, q);
      break;
    case 142:
      LaunchShape<1, 4, 2>(out_kind, grid, stream, q);
      break;
    case 114:
      LaunchShape<1, 1, 4>(out_kind, grid, stream, q);
      break;
    case 124:
      LaunchShape<1, 2, 4>(out_kind, grid, stream, q);
      break;
    case 221:
      LaunchShape<2, 2, 1>(out_kind, grid, stream, q);
      break;
    case 212:
      LaunchShape<2, 1, 2>(out_kind, grid, stream, q);
      break;
    case 222:
      LaunchShape<2, 2, 2>(out_kind, grid, stream, q);
      break;
    case 214:
      LaunchShape<2, 1, 4>(out_kind, grid, stream, q);
      break;
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace pl
