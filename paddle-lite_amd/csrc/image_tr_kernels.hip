// Image MFMA with transposing LDS reads: int8 sparse 1x1 convolution for
// feature maps whose rows are 4 (mod 8) bytes long (14 x 14, 10 x 10, 6 x 10 ...)
// and small enough that one image ([K x H*W] int8) fits the LDS of a CU.
//
// One workgroup of eight wavefronts computes 128 output rows of one image.
//   * The image is copied into LDS exactly as it lies in memory ([channel][H*W],
//     16-byte direct loads, no registers) and is never rearranged.  The matrix
//     cores want, per lane, 16 channels of one position; ds_read_b64_tr_b8
//     delivers that from the channel-major copy: within 16 lanes, lane j byte b
//     receives byte j % 8 of what lane 2 b + j / 8 addressed.  Two such reads
//     make one operand of v_mfma_i32_16x16x64_i8 (64 channels x 16 positions).
//   * The read wants 8-byte aligned addresses (the low three address bits are
//     ignored).  With rows of 4 (mod 8) bytes the rows of even channels start
//     on 8-byte boundaries and the rows of odd channels 4 bytes off, so an
//     aligned read covers positions 8 u .. 8 u + 7 of an even channel and
//     8 u + 4 .. 8 u + 11 of an odd one.  Every k-step therefore takes channels
//     of one parity (the order of the channels inside a dot product is free:
//     integer sums are exact, and the weight tiles are laid out to match), and
//     the two parities are accumulated separately, one position quad apart.
//   * Channels of one k-step and half wavefront are four apart: with rows of
//     an odd number of dwords their 16-byte pieces then fall into distinct
//     LDS banks (no bank conflicts measured).
//   * Positions are the rows of the matrix product and output rows its
//     columns: a lane ends with four neighbouring positions of one output row,
//     16 bytes of fp32.  The sums of the shifted parity sit one lane group
//     (one quad) off; they go through a small LDS buffer and come back from
//     the neighbouring group.
//   * A wavefront owns 16 output rows rho, rho + 4, rho + 8 ... (rho = row mod 4)
//     and all positions.  Rows of one class start at the same offset inside a
//     64-byte sector of the fp32 output, so the class's windows of 16 positions
//     are placed on sector boundaries.  Stores of 64 bytes per row reach only
//     two thirds of the rate of whole 128-byte lines on this device (measured
//     with a store-only kernel of the same shape: 8.6 against 5.3 us for the
//     25.7 MB of 64 x 512 x 14 x 14 floats), so two windows of a row leave
//     together: odd windows are multiplied with the rows of the tile exchanged
//     in pairs, which puts the second half of a row's line into the lane next
//     to the one that holds the first half, and one store covers eight rows x
//     128 bytes, written through (sc1 nt).  The pieces at the two ends of a
//     row that share a line with a neighbouring row are stored plainly.
//
// Reference semantics: out = act(fmaf(float(acc), scale, bias)) per output,
// int32 accumulation over all channels (sparse_conv_impl.cc:1661-1685 computes
// the same sum over the nonzeros only; zeros add nothing to an integer sum).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "epilogue.h"
#include "kernarg_head.h"
#include "launch_lds.h"
#include "sparse_conv_kernels.h"

namespace pl {
namespace {

using epilogue::ActivateT;
using epilogue::ActQuantF;
using epilogue::DispatchAct;
using epilogue::TruncPackI8x4;

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
#define PL_LDS __attribute__((address_space(3)))

constexpr int kFrontPad = 256;    // windows reach up to 16 bytes in front of the first channel row
constexpr int kBackPad = 128;     // and up to 96 bytes behind the last one
constexpr int kStageBytes = 5120; // per wavefront: the shifted sums of five windows, 16 rows x 64 bytes each

// 8 channels x 16 positions for a group of 16 lanes (see the file comment).
__device__ __forceinline__ v2i ReadTr8(PL_LDS char* lds, int byte_offset) { return __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<PL_LDS v2i*>(lds + byte_offset)); }

// 16 bytes written through to memory as streaming data; wave-uniform base plus unsigned 32-bit lane offset.
// The wait state keeps the data registers intact until the store has read them.
__device__ __forceinline__ void StoreThrough128(u4 v, char* base, uint32_t off) { asm volatile("global_store_dwordx4 %0, %1, %2 sc1 nt\n s_nop 1" ::"v"(off), "v"(v), "s"(base) : "memory"); }

// KS2 = K / 128: k-steps per channel parity.  HW: H*W when known at compile
// time (LDS offsets become immediates), else 0.
template <int KS2, int OUT, int HW>
__global__ void __launch_bounds__(512) ImageTrKernel(PL_HEAD_PARAMS, const ImageMfmaParams block) {
  const ImageMfmaParams p = WithHead(block, PL_HEAD_ARGS);
  extern __shared__ uint4 lds_raw[];
  PL_LDS char* img = (PL_LDS char*)lds_raw + kFrontPad;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // a contiguous range of work items per XCD, the row groups of one image next to each other
  const int item = (int)(blockIdx.x & 7u) * p.per_xcd + (int)(blockIdx.x >> 3);
  if (item >= p.items) return;
  const int n = item / p.row_groups, rg = item - n * p.row_groups;
  const int rho = wave & 3, j = (wave >> 2) & 1;
  const int hw = HW ? HW : p.hw;

  // activations: every wavefront moves a contiguous eighth of the image straight into LDS
  {
    const int per_wave = (p.K >> 3) * hw;  // a multiple of 16 (K is a multiple of 128, hw of 4)
    const int8_t* src = p.x + (size_t)n * p.K * hw + (size_t)wave * per_wave + lane * 16;
    PL_LDS char* dst = img + wave * per_wave;
    for (int t = 0; t < p.dma_full; ++t)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + t * 1024), (PL_LDS void*)(dst + t * 1024), 16, 0, 0);
    if (lane < p.dma_rem_lanes)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + p.dma_full * 1024), (PL_LDS void*)(dst + p.dma_full * 1024), 16, 0, 0);
  }

  // Placement of the class's windows.  A row of the class starts qoff position quads into a sector.
  constexpr bool PAIR = OUT != kOutI8;  // fp32 / int32 rows leave as whole 128-byte lines made of two windows
  const int qoff = p.align ? ((rho * (hw >> 2)) & 3) : 0;
  const int a0 = (16 - 4 * qoff) & 15;   // first position of the windows, mod 16
  const int par_d = (a0 >> 2) & 1;       // channel parity whose aligned reads start at a0 (mod 8)
  const int par_s = par_d ^ 1;           // the other parity is read four positions to the left

  const int pn = lane & 15, kq = lane >> 4, odd = pn & 1;
  // Weights of the wavefront's row tile: k-steps of the direct and of the shifted parity.  Positions are the
  // rows of the matrix product and output rows its columns: lane (pn, kq) ends with positions 4 kq .. 4 kq + 3
  // of a window for the row its weight operand holds.  Even windows take the tile as it is (lane pn = row
  // pn), odd windows take it with neighbouring rows exchanged (lane pn = row pn ^ 1): the two halves of a
  // 128-byte line of an output row (two windows) then sit in neighbouring lanes and leave in one store.
  v4i a_d[KS2], a_s[KS2], b_d[KS2], b_s[KS2];
  {
    const v4i* wt = static_cast<const v4i*>(p.wtiles) + ((size_t)((rg * 4 + rho) * 2 + j) * (2 * KS2)) * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < KS2; ++ks) {
      a_d[ks] = wt[(2 * ks + par_d) * 64];
      a_s[ks] = wt[(2 * ks + par_s) * 64];
    }
    // the tile with neighbouring rows exchanged: every lane takes its neighbour's registers
#pragma unroll
    for (int ks = 0; ks < KS2; ++ks) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        b_d[ks][c] = PAIR ? __builtin_amdgcn_mov_dpp(a_d[ks][c], 0xB1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, true) : a_d[ks][c];
        b_s[ks][c] = PAIR ? __builtin_amdgcn_mov_dpp(a_s[ks][c], 0xB1, 0xf, 0xf, true) : a_s[ks][c];
      }
    }
  }
  // rows of the tile, relative to the row group: the even row and the odd row of the lane's pair
  const int rowA = rho + 4 * (16 * j + (pn & ~1)), rowB = rho + 4 * (16 * j + (pn | 1));
  const int row_own = rho + 4 * (16 * j + pn);
  float scA = 0.f, biA = 0.f, scB = 0.f, biB = 0.f;
  if (OUT != kOutAcc32) {
    scA = p.scale[rg * 128 + (PAIR ? rowA : row_own)];
    biA = p.bias[rg * 128 + (PAIR ? rowA : row_own)];
    scB = p.scale[rg * 128 + (PAIR ? rowB : row_own)];
    biB = p.bias[rg * 128 + (PAIR ? rowB : row_own)];
  }
  // everything requested so far has arrived (the direct loads included), in every wavefront
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();

  // Addresses of the transposing reads.  Lane s of a group of 16 lanes supplies byte s / 2 of the
  // operand (channel) for the positions of run s % 2 (8 positions each); group g = lane / 16 holds
  // channels 4 t + 2 (g / 2) + parity + 64 r + 128 ks, t = 8 (g % 2) + s / 2, r = first / second read.
  const int lane_off = (4 * (8 * (kq & 1) + (pn >> 1)) + 2 * (kq >> 1)) * hw + 8 * (pn & 1);
  const int step_r = 64 * hw, step_ks = 128 * hw;

  const int T0 = a0 > 0 ? -1 : 0;
  const int T1 = (hw - 1 - a0) >> 4;  // last window that holds a position of the row
  const int NW = T1 - T0 + 1;         // windows to store; window NW is computed for its shifted sums only
  // read addresses of window 0; 16 bytes further per window
  int rd_d = lane_off + par_d * hw + a0 + 16 * T0;
  int rd_s = lane_off + par_s * hw + a0 - 4 + 16 * T0;

  // The sums over the channels of the shifted parity lie one position quad to the left of the direct
  // ones: lane group kq needs what group kq + 1 holds, and group 3 what group 0 holds for the next
  // window (where the rows of a pair sit the other way round).  They go through a staging buffer of the
  // wavefront, [window of the group][lane group][lane] x 16 bytes.
  PL_LDS char* stage = img + p.K * hw + kBackPad + wave * kStageBytes;
  PL_LDS char* st_wr = stage + lane * 16;
  PL_LDS char* st_rd = stage + (kq < 3 ? ((kq + 1) * 16 + pn) * 16 : 1024 + (PAIR ? (pn ^ 1) : pn) * 16);

  constexpr int kElem = OUT == kOutI8 ? 1 : 4;
  // first byte of the row group's output; pos0 = first position of window 0
  char* obase = static_cast<char*>(p.out) + ((size_t)n * p.M + (size_t)rg * 128) * hw * kElem;
  int pos0 = a0 + 16 * T0;
  // fp32 / int32: a store covers the pair of windows (w - 1, w): even lanes hold window w - 1, odd lanes
  // window w, of the pair's even row (w odd) or odd row (w even); lane offsets inside that line
  const uint32_t offA = (uint32_t)((rowA * hw) * 4 + 64 * odd + 16 * kq), offB = (uint32_t)((rowB * hw) * 4 + 64 * odd + 16 * kq);
  const uint32_t off8 = (uint32_t)(row_own * hw + 4 * kq);  // int8: the lane's own row and quad
  v4i prev = v4i{0, 0, 0, 0};  // sums of the window before the one in hand

  DispatchAct(OUT == kOutAcc32 ? 0 : p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    auto finish = [&](const v4i& acc, float sc, float bi) {
      if (OUT == kOutI8)
        return u4{TruncPackI8x4(ActQuantF<ACT>(__builtin_fmaf((float)acc[0], sc, bi), p.act), ActQuantF<ACT>(__builtin_fmaf((float)acc[1], sc, bi), p.act),
                                ActQuantF<ACT>(__builtin_fmaf((float)acc[2], sc, bi), p.act), ActQuantF<ACT>(__builtin_fmaf((float)acc[3], sc, bi), p.act)), 0u, 0u, 0u};
      if (OUT == kOutAcc32) return u4{(uint32_t)acc[0], (uint32_t)acc[1], (uint32_t)acc[2], (uint32_t)acc[3]};
      return u4{__float_as_uint(ActivateT<ACT>(__builtin_fmaf((float)acc[0], sc, bi), p.act)), __float_as_uint(ActivateT<ACT>(__builtin_fmaf((float)acc[1], sc, bi), p.act)),
                __float_as_uint(ActivateT<ACT>(__builtin_fmaf((float)acc[2], sc, bi), p.act)), __float_as_uint(ActivateT<ACT>(__builtin_fmaf((float)acc[3], sc, bi), p.act))};
    };
    // window w (its sums in acc; ODD = w odd) is finished: the pair (w - 1, w) is stored
    auto emit = [&](auto odd_c, const v4i& acc) {
      constexpr int ODD = decltype(odd_c)::value;
      if (!PAIR) {
        const int pos = pos0 + 4 * kq;
        const u4 bits = finish(acc, scA, biA);
        if (pos >= 0 && pos < hw) *reinterpret_cast<uint32_t*>(obase + pos0 + off8) = bits.x;
      } else {
        // even lanes: window w - 1, odd lanes: window w
        v4i sel;
#pragma unroll
        for (int i = 0; i < 4; ++i) sel[i] = odd ? acc[i] : prev[i];
        const u4 bits = ODD ? finish(sel, scA, biA) : finish(sel, scB, biB);
        const int first = pos0 - 16;                      // first position of window w - 1
        const int pos = first + 16 * odd + 4 * kq;        // the lane's quad
        char* line = obase + __builtin_amdgcn_readfirstlane(first * 4);
        const uint32_t off = ODD ? offA : offB;
        if (first >= 0 && first + 32 <= hw) StoreThrough128(bits, line, off);
        else if (pos >= 0 && pos < hw) *reinterpret_cast<u4*>(line + off) = bits;
        prev = acc;
      }
      pos0 += 16;
    };
    // A group of G windows: direct sums of G windows and shifted sums of G + 1 windows, channels outermost
    // (the operands of the next k-step are requested before the current one is multiplied), then the
    // shifted sums through the staging buffer, then epilogue and stores.
    int left = NW;
    auto group = [&](auto g_c) {
      constexpr int G = decltype(g_c)::value;
      v2i od[2][G][2], os[2][G + 1][2];
      v4i d[G], s[G + 1];
#pragma unroll
      for (int i = 0; i < G; ++i) d[i] = v4i{0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i <= G; ++i) s[i] = v4i{0, 0, 0, 0};
      auto request = [&](int buf, int ks) {
#pragma unroll
        for (int i = 0; i <= G; ++i) {
#pragma unroll
          for (int r = 0; r < 2; ++r) {
            os[buf][i][r] = ReadTr8(img, rd_s + 16 * i + ks * step_ks + r * step_r);
            if (i < G) od[buf][i][r] = ReadTr8(img, rd_d + 16 * i + ks * step_ks + r * step_r);
          }
        }
      };
      request(0, 0);
#pragma unroll
      for (int ks = 0; ks < KS2; ++ks) {
        if (ks + 1 < KS2) request((ks + 1) & 1, ks + 1);
#pragma unroll
        for (int i = 0; i <= G; ++i) {
          const int b = ks & 1;
          s[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{os[b][i][0].x, os[b][i][0].y, os[b][i][1].x, os[b][i][1].y}, (i & 1) ? b_s[ks] : a_s[ks], s[i], 0, 0, 0);
          if (i < G) d[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{od[b][i][0].x, od[b][i][0].y, od[b][i][1].x, od[b][i][1].y}, (i & 1) ? b_d[ks] : a_d[ks], d[i], 0, 0, 0);
        }
      }
      rd_d += 16 * G;
      rd_s += 16 * G;
#pragma unroll
      for (int i = 0; i <= G; ++i) *reinterpret_cast<PL_LDS v4i*>(st_wr + i * 1024) = s[i];
      v4i sh[G];
#pragma unroll
      for (int i = 0; i < G; ++i) sh[i] = *reinterpret_cast<PL_LDS v4i*>(st_rd + i * 1024);
#pragma unroll
      for (int i = 0; i < G; ++i) {
        const v4i acc = d[i] + sh[i];
        if (i & 1) emit(std::integral_constant<int, 1>(), acc);
        else emit(std::integral_constant<int, 0>(), acc);
      }
    };
    for (; left >= 4; left -= 4) {
      group(std::integral_constant<int, 4>());
    }
    if (left >= 2) {
      group(std::integral_constant<int, 2>());
      left -= 2;
    }
    if (left >= 1) {
      group(std::integral_constant<int, 1>());
      // the group started at an even window, so the window after it is odd
      if (PAIR) emit(std::integral_constant<int, 1>(), v4i{0, 0, 0, 0});
    } else if (PAIR) {
      emit(std::integral_constant<int, 0>(), v4i{0, 0, 0, 0});
    }
  });
}

template <int OUT>
hipError_t ByKs(const ImageMfmaParams& q, dim3 grid, size_t lds, hipStream_t s) {
  const dim3 block(512);
  if (q.hw == 196) {
    switch (q.K / 128) {
      case 1:
        return LaunchWithHead(ImageTrKernel<1, OUT, 196>, grid, block, lds, s, q);
      case 2:
        return LaunchWithHead(ImageTrKernel<2, OUT, 196>, grid, block, lds, s, q);
      case 4:
        return LaunchWithHead(ImageTrKernel<4, OUT, 196>, grid, block, lds, s, q);
      default:
        return hipErrorInvalidValue;
    }
  }
  switch (q.K / 128) {
    case 1:
      return LaunchWithHead(ImageTrKernel<1, OUT, 0>, grid, block, lds, s, q);
    case 2:
      return LaunchWithHead(ImageTrKernel<2, OUT, 0>, grid, block, lds, s, q);
    case 4:
      return LaunchWithHead(ImageTrKernel<4, OUT, 0>, grid, block, lds, s, q);
    default:
      return hipErrorInvalidValue;
  }
}

size_t LdsBytes(int K, int hw) { return (size_t)kFrontPad + (size_t)K * hw + kBackPad + 8 * (size_t)kStageBytes; }

}  // namespace

bool ImageTrMfmaFits(int M, int K, int hw) {
  if (M <= 0 || M % 128 != 0) return false;
  if (K != 128 && K != 256 && K != 512) return false;
  if (hw < 20 || hw > 252 || hw % 8 != 4) return false;
  return LdsBytes(K, hw) <= (size_t)kMaxLdsBytes;
}

hipError_t LaunchImageTrMfma(int out_kind, const ImageMfmaParams& p, hipStream_t stream) {
  if (p.batch <= 0) return hipSuccess;
  if (!ImageTrMfmaFits(p.M, p.K, p.hw)) return hipErrorInvalidValue;
  if (reinterpret_cast<uintptr_t>(p.x) % 16 != 0 || reinterpret_cast<uintptr_t>(p.out) % 16 != 0) return hipErrorInvalidValue;
  ImageMfmaParams q = p;
  q.qpi = p.hw / 4;
  q.kgs = 0;
  q.row_groups = p.M / 128;
  const int64_t items = (int64_t)p.batch * q.row_groups;
  if (items > (1 << 28)) return hipErrorInvalidValue;
  q.items = (int)items;
  q.per_xcd = (q.items + 7) / 8;
  const int per_wave = (p.K / 8) * p.hw;
  q.dma_full = per_wave / 1024;
  q.dma_rem_lanes = (per_wave % 1024) / 16;
  q.align = out_kind != kOutI8;
  const dim3 grid(8u * (uint32_t)q.per_xcd);
  switch (out_kind) {
    case kOutF32:
      return ByKs<kOutF32>(q, grid, LdsBytes(p.K, p.hw), stream);
    case kOutI8:
      return ByKs<kOutI8>(q, grid, LdsBytes(p.K, p.hw), stream);
    case kOutAcc32:
      return ByKs<kOutAcc32>(q, grid, LdsBytes(p.K, p.hw), stream);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace pl
