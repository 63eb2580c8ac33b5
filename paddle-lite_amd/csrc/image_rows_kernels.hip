// Image MFMA, one row tile per wavefront: int8 sparse 1x1 convolution for feature maps of which one image
// ([K x H*W] int8) fits the LDS of a CU.  Same work split over the chip as image_mfma_kernels.hip (one workgroup
// of eight wavefronts per image and 128 output rows, the image held in LDS as 16-byte cells of 16 channels of
// one position), with three differences that were each measured on 64 x 512 -> 512 @14x14, fp32 output:
//
//   * The image goes through registers, not through an LDS landing area.  A lane loads the dword (four
//     positions) of one position quad for each of 16 consecutive channels, transposes the 16 x 4 bytes with
//     two stages of v_perm_b32 and writes four cells.  LDS then takes the image once (writes run at about
//     71 bytes per clock per CU, a third of the read rate); landing it by direct loads and regrouping it in place
//     writes it twice and was 0.3 us slower.  The weight tiles of two k-steps are requested behind every
//     regrouped channel group, so that they queue up behind the image and arrive in the order the
//     multiplication uses them.
//   * A wavefront owns ONE tile of 16 output rows and all positions (the other kernel gives a pair of
//     wavefronts two tiles and splits the positions).  Every wavefront then loads only its own 8 KB of
//     weights - half the weight traffic of the workgroup - and every unit of work is small: a window of 64
//     positions is 32 matrix instructions, after which its 16 x 64 outputs are finished (scale, bias,
//     activation) and stored between the k-steps of the next window, where the vector ALU would idle.
//   * The rows of a tile are 8 apart (row = w + 8 m for wavefront w).  A row of 196 fp32 outputs is 784
//     bytes = 6 1/8 lines of 128 bytes, so rows 8 apart start at the same offset inside a line; the
//     wavefront shifts its windows left by that offset and every 256-byte piece it stores is two whole
//     lines.  With rows 4 apart pieces start on 64-byte boundaries only and half of them straddle lines;
//     partially written lines cost the memory system a second access (9.24 -> 9.09 us).
//
// Wavefront w starts with window w mod (windows per row) and goes round from there, so that at any time all
// parts of the rows are being written rather than one column of the output (all wavefronts ascending 9.9 - 10.4 us,
// the upper four descending 9.23, going round 9.09 in one run).
//
// A second kernel (ImageRowsDwKernel) runs the int8 depthwise 3 x 3 layer that follows such a pointwise layer in
// a MobileNet in the same launch: the tile of a wavefront is 16 output channels times all positions, i.e. 16 whole
// planes of the depthwise layer.  With int8 output the epilogue writes them to the wavefront's own LDS instead of
// global memory, and behind its last window the wavefront computes the depthwise layer on them (DwStage, no
// barrier: the planes are private to the wavefront).  14 x 14 maps, padding 1, stride 1 or 2.
//
// Reference semantics: out = act(fmaf(float(acc), scale, bias)) per output, int32 accumulation over all
// channels (sparse_conv_impl.cc:1661-1685 computes the same sum over the nonzeros only; zeros add nothing to
// an integer sum).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "dw_row_item.h"
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

typedef int v4i __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

// what the image and weight loads need arrives in registers
PL_IN_HEAD(ImageMfmaParams, x);
PL_IN_HEAD(ImageMfmaParams, out);
PL_IN_HEAD(ImageMfmaParams, wtiles);
PL_IN_HEAD(ImageMfmaParams, K);
PL_IN_HEAD(ImageMfmaParams, hw);
PL_IN_HEAD(ImageMfmaParams, items);
PL_IN_HEAD(ImageMfmaParams, per_xcd);
PL_IN_HEAD(ImageMfmaParams, row_groups);
PL_IN_HEAD(ImageMfmaParams, pitch);
PL_IN_HEAD(ImageMfmaParams, slabs);

constexpr int kRowStride = 8;  // rows of a tile: w + 8 m
// Output kind of the kernel that runs the following depthwise layer itself: int8 like kOutI8, written to the
// wavefront's own planes in LDS (one plane of H x W bytes per row of its tile) instead of global memory.
constexpr int kOutPlanes = 3;
template <int OUT>
constexpr int kPlaneStride = OUT == kOutPlanes ? 1 : kRowStride;  // rows of the tile are this many rows apart where they are stored
__device__ __forceinline__ void StoreLds(uint32_t v, char* p) {
  *reinterpret_cast<__attribute__((address_space(3))) uint32_t*>(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p))) = v;
}

// 16 bytes stored as streaming data (nt) at a wave-uniform base plus an unsigned 32-bit lane offset (no 64-bit
// address arithmetic per store).  Measured on the metric shape with this kernel's whole-line pieces: nt 8.93 us,
// sc1 nt 9.05, sc0 sc1 nt 9.06, sc1 10.9, no policy 11.9.  The wait state after the store keeps the data registers
// intact until the store has read them (the compiler does not see a store inside the assembly statement).
__device__ __forceinline__ void StoreStreaming(u4 v, char* base, uint32_t off) {
  asm volatile("global_store_dwordx4 %0, %1, %2 nt\n s_nop 1" ::"v"(off), "v"(v), "s"(base) : "memory");
}
// Plain stores name the global address space: the output pointer passes through scalar registers (Uniform), where
// the compiler loses track of where it points, and a store through a generic pointer is a flat store, which
// also counts as an LDS operation in the wavefront's wait counters.
__device__ __forceinline__ void StorePlain(u4 v, void* p) { *reinterpret_cast<__attribute__((address_space(1))) u4*>(reinterpret_cast<uintptr_t>(p)) = v; }
__device__ __forceinline__ void StorePlain(uint32_t v, void* p) { *reinterpret_cast<__attribute__((address_space(1))) uint32_t*>(reinterpret_cast<uintptr_t>(p)) = v; }
// A pointer that is the same in every lane, as a scalar register pair (the halves are taken as unsigned: a low
// half with its top bit set must not be sign-extended into the high half).
__device__ __forceinline__ char* Uniform(char* p) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a), hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
  return reinterpret_cast<char*>(((uint64_t)hi << 32) | (uint64_t)lo);
}

struct Lane {
  int n;   // column of a 16x16 tile
  int kq;  // quarter of the wavefront: channel group of an operand, rows 4 kq .. 4 kq + 3 of a result
};

template <int OUT, int ACT>
__device__ __forceinline__ u4 Finish4(int a0, int a1, int a2, int a3, float s, float b, const DevAct& act) {
  if (OUT == kOutAcc32) return u4{(uint32_t)a0, (uint32_t)a1, (uint32_t)a2, (uint32_t)a3};
  const float v0 = __builtin_fmaf((float)a0, s, b), v1 = __builtin_fmaf((float)a1, s, b), v2 = __builtin_fmaf((float)a2, s, b), v3 = __builtin_fmaf((float)a3, s, b);
  if (OUT == kOutI8 || OUT == kOutPlanes) return u4{TruncPackI8x4(ActQuantF<ACT>(v0, act), ActQuantF<ACT>(v1, act), ActQuantF<ACT>(v2, act), ActQuantF<ACT>(v3, act)), 0u, 0u, 0u};
  return u4{__float_as_uint(ActivateT<ACT>(v0, act)), __float_as_uint(ActivateT<ACT>(v1, act)), __float_as_uint(ActivateT<ACT>(v2, act)), __float_as_uint(ActivateT<ACT>(v3, act))};
}

// Row 4 kq + i of a window's results (positions 4 q .. 4 q + 3 per lane): epilogue and store.  `partial`: the
// lane's line is shared with the end of the previous output row and merges in L2 (plain store).
template <int OUT, int ACT>
__device__ __forceinline__ void StoreRow(const v4i (&acc)[4], int i, float sc, float bi, const DevAct& act, char* __restrict__ orow, int pitch, int q, bool partial, Lane ln) {
  constexpr int kElem = (OUT == kOutI8 || OUT == kOutPlanes) ? 1 : 4;
  const u4 v = Finish4<OUT, ACT>(acc[0][i], acc[1][i], acc[2][i], acc[3][i], sc, bi, act);
  // at most 128 rows of at most 256 four-byte positions behind orow: the offset fits 32 bits; it is negative only
  // for the quads in front of a row, which are not stored
  const int off = ((kPlaneStride<OUT> * (4 * ln.kq + i)) * pitch + 4 * q) * kElem;
  if (OUT == kOutPlanes) {
    if (q >= 0) StoreLds(v.x, orow + off);
  } else if (OUT == kOutI8) {
    if (q >= 0) StorePlain(v.x, orow + off);
  } else if (partial) {
    if (q >= 0) StorePlain(v, orow + off);
  } else {
    StoreStreaming(v, orow, (uint32_t)off);
  }
}

// LDS of a wavefront behind the image's cells when the depthwise layer follows: its 16 planes of 14 x 14 int8
// (16 bytes of slack in front, 48 behind: the rows are read as aligned dwords around them), then the planes of
// the depthwise output.
constexpr int kPlaneInBytes = 16 + 16 * 196 + 48, kPlaneBufBytes = kPlaneInBytes + 16 * 196;

// The depthwise layer on the wavefront's planes: one output row of one plane per lane and pass (dw_row_item.h),
// outputs collected plane-major in LDS, then stored: a plane of the tile's row m is channel row0 + 8 m.
template <int STRIDE>
__device__ __forceinline__ void DwStage(const DwConvParams& d, char* planes_in, char* planes_out, int n, int M, int row0, int lane) {
  constexpr int NOUT = STRIDE == 1 ? 14 : 7;
  constexpr int oh = NOUT, ow = NOUT;  // 14 x 14 planes, padding 1
  constexpr int items = 16 * oh, passes = (items + 63) / 64;
  dwrow::DwRowStage st;
  st.lds_in = planes_in - 16;
  st.in_base = 0;
  // filter rows, scale and bias of every pass's channel first: one memory latency for all passes
  uint32_t wrow[passes][3];
  float sc[passes], bi[passes];
#pragma unroll
  for (int t = 0; t < passes; ++t) {
    const int it = min(64 * t + lane, items - 1);
    const int c = row0 + kRowStride * (it / oh);
    wrow[t][0] = d.wpack[4 * c];
    wrow[t][1] = d.wpack[4 * c + 1];
    wrow[t][2] = d.wpack[4 * c + 2];
    sc[t] = d.scale[c];
    bi[t] = d.bias[c];
  }
  DispatchAct(d.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int t = 0; t < passes; ++t) {
      const int item = 64 * t + lane;
      const bool live = item < items;
      const int it = live ? item : items - 1;
      const int m = it / oh, oy = it - m * oh;
      dwrow::DwRowItemWith<STRIDE, NOUT, kOutI8, ACT, 14>(d, st, (uint32_t)m, wrow[t], sc[t], bi[t], oy, live, planes_out + it * ow);
    }
  });
  const int plane_bytes = oh * ow;
  char* obase = static_cast<char*>(d.out) + ((size_t)n * M + row0) * plane_bytes;
  if ((plane_bytes & 3) == 0) {
    const int per = plane_bytes >> 2;
    for (int k = lane; k < 16 * per; k += 64) {
      const int m = k / per, j = k - m * per;
      StorePlain(*reinterpret_cast<const uint32_t*>(planes_out + 4 * k), obase + (size_t)(kRowStride * m) * plane_bytes + 4 * j);
    }
  } else {
    for (int k = lane; k < 16 * plane_bytes; k += 64) {
      const int m = k / plane_bytes, j = k - m * plane_bytes;
      *reinterpret_cast<__attribute__((address_space(1))) char*>(reinterpret_cast<uintptr_t>(obase + (size_t)(kRowStride * m) * plane_bytes + j)) = planes_out[k];
    }
  }
}

// One window of 16 position quads times the wavefront's row tile.  When EPI, the four rows of the previous
// window (accumulators accp, first quad qp) are finished and stored between the k-steps, one row per KS / 4
// k-steps (all of them behind the last k-step when KS < 4).
template <int KS, int OUT, int ACT, bool EPI>
__device__ __forceinline__ void Window(const uint4* __restrict__ xt, int kgs, int cps, int q0, const v4i (&a)[KS], v4i (&acc)[4], const v4i (&accp)[4], int qp, bool partialp, const float (&sc)[4],
                                       const float (&bi)[4], const DevAct& act, char* __restrict__ orow, int pitch, Lane ln) {
  const uint4* bbase = xt + ln.kq * kgs + (q0 + ln.n);  // + ks * 4 * kgs + c * cps
#pragma unroll
  for (int c = 0; c < 4; ++c) acc[c] = v4i{0, 0, 0, 0};
  // operand cells in flight ahead of the multiply: two k-steps where the multiply is what the wavefront waits for
  // (int8 output), one where it hides behind the stores (8.13 against 8.17 us on the metric shape; three: 8.27)
  constexpr int PF = (OUT == kOutI8 || OUT == kOutPlanes) ? 2 : 1;
  constexpr int kStepsPerRow = KS >= 4 ? KS / 4 : 1;
  uint4 bq[PF + 1][4];
#pragma unroll
  for (int d = 0; d < PF; ++d)
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if (d < KS) bq[d][c] = bbase[d * 4 * kgs + c * cps];
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (ks + PF < KS) {
#pragma unroll
      for (int c = 0; c < 4; ++c) bq[(ks + PF) % (PF + 1)][c] = bbase[(ks + PF) * 4 * kgs + c * cps];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint4 u = bq[ks % (PF + 1)][c];
      acc[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[ks], v4i{(int)u.x, (int)u.y, (int)u.z, (int)u.w}, acc[c], 0, 0, 0);
    }
    if (EPI && ks % kStepsPerRow == 0 && ks / kStepsPerRow < 4) {
      const int i = ks / kStepsPerRow;
      StoreRow<OUT, ACT>(accp, i, sc[i], bi[i], act, orow, pitch, qp + ln.n, partialp && ln.n < kRowStride, ln);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  if (EPI && KS < 4) {
#pragma unroll
    for (int i = KS; i < 4; ++i) StoreRow<OUT, ACT>(accp, i, sc[i], bi[i], act, orow, pitch, qp + ln.n, partialp && ln.n < kRowStride, ln);
  }
}

// QPI: quads per image when known at compile time (49 = 14 x 14 maps), else 0: the LDS offsets of the cells
// then become immediates.
//
// The head of the parameter block arrives in registers (kernarg_head.h): the image loads do not wait for a
// load of the kernel arguments from memory (8.36 -> 8.10 us on the metric shape).
//
// dw (kOutPlanes only): the depthwise layer that follows; the wavefront then keeps its 16 output planes in LDS
// and runs that layer on them (DwStage below).
//
// SLAB: a work item takes one slab of hw positions of a larger map (p.pitch positions per channel, p.slabs slabs
// per image): the channel rows of the input and the rows of the output are then p.pitch apart, not hw.
template <int KS, int OUT, int QPI, int DW_STRIDE = 0, bool SLAB = false>
__device__ __forceinline__ void RowsBody(const ImageMfmaParams& p, uint4* lds_raw, const DwConvParams* dw) {
  // shifted windows read up to seven cells in front of a row of cells
  uint4* xt = lds_raw + 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // a contiguous range of work items per XCD, the row groups of one image next to each other
  const int item = (int)(blockIdx.x & 7u) * p.per_xcd + (int)(blockIdx.x >> 3);
  if (item >= p.items) return;
  const int ns = item / p.row_groups, rg = item - ns * p.row_groups;
  const int n = SLAB ? ns / p.slabs : ns, slab = SLAB ? ns - n * p.slabs : 0;
  const int hw = p.hw, pitch = SLAB ? p.pitch : hw;
  const int qpi = QPI ? QPI : hw >> 2, kgs = QPI ? (4 * QPI + 15) / 16 * 16 : ((hw + 15) >> 4) << 4;
  const int cps = qpi;  // cells of position c of every quad lie qpi cells apart
  constexpr int NKG = 4 * KS, BPW = NKG / 8;
  static_assert(NKG % 8 == 0, "channel groups are dealt evenly to the eight wavefronts");

  // the image: dword (channel, quad) of the wavefront's channel groups, lane = quad
  uint32_t r[BPW][16];
  {
    // one address per channel group, the channel's offset in the instruction (16 rows of at most 256 bytes)
    const char* ximg = reinterpret_cast<const char*>(p.x) + (size_t)n * p.K * pitch + slab * hw + lane * 4;
    const int row_bytes = SLAB ? pitch : (QPI ? 4 * QPI : hw);
    if (lane < qpi) {
#pragma unroll
      for (int u = 0; u < BPW; ++u) {
        const char* group = ximg + (size_t)((wave * BPW + u) * 16) * row_bytes;
#pragma unroll
        for (int i = 0; i < 16; ++i) r[u][i] = *reinterpret_cast<const uint32_t*>(group + i * row_bytes);
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // every channel group becomes four cells per quad; the weights of KS / BPW k-steps are requested behind it
  char* lbase = reinterpret_cast<char*>(xt);
  v4i a[KS];
  const v4i* wt = static_cast<const v4i*>(p.wtiles) + ((size_t)(rg * 8 + wave) * KS) * 64 + lane;
#pragma unroll
  for (int u = 0; u < BPW; ++u) {
    if (lane < qpi) {
      // Two stages of byte permutes.  The second stage is done cell by cell so that the four dwords of a
      // cell (one per block of four channels) are produced next to each other, where the 16-byte write
      // wants them.
      uint32_t lo[4][2], hi[4][2];
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        lo[b4][0] = __builtin_amdgcn_perm(r[u][4 * b4 + 1], r[u][4 * b4], 0x05010400u);      // positions 0, 1 of channels 4 b4, 4 b4 + 1
        hi[b4][0] = __builtin_amdgcn_perm(r[u][4 * b4 + 1], r[u][4 * b4], 0x07030602u);      // positions 2, 3
        lo[b4][1] = __builtin_amdgcn_perm(r[u][4 * b4 + 3], r[u][4 * b4 + 2], 0x05010400u);  // the same of channels 4 b4 + 2, 4 b4 + 3
        hi[b4][1] = __builtin_amdgcn_perm(r[u][4 * b4 + 3], r[u][4 * b4 + 2], 0x07030602u);
      }
      uint4* cells = reinterpret_cast<uint4*>(lbase + (wave * BPW + u) * (kgs * 16)) + lane;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
        uint4 cell;
        cell.x = __builtin_amdgcn_perm((c & 2) ? hi[0][1] : lo[0][1], (c & 2) ? hi[0][0] : lo[0][0], sel);
        cell.y = __builtin_amdgcn_perm((c & 2) ? hi[1][1] : lo[1][1], (c & 2) ? hi[1][0] : lo[1][0], sel);
        cell.z = __builtin_amdgcn_perm((c & 2) ? hi[2][1] : lo[2][1], (c & 2) ? hi[2][0] : lo[2][0], sel);
        cell.w = __builtin_amdgcn_perm((c & 2) ? hi[3][1] : lo[3][1], (c & 2) ? hi[3][0] : lo[3][0], sel);
        cells[c * qpi] = cell;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = u * (KS / BPW); ks < (u + 1) * (KS / BPW); ++ks) a[ks] = wt[ks * 64];
    __builtin_amdgcn_sched_barrier(0);
  }
  Lane ln;
  ln.n = lane & 15;
  ln.kq = lane >> 4;
  const int row0 = rg * 128 + wave;  // the wavefront's rows: row0 + 8 m, m = 0 .. 15
  float sc[4], bi[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    sc[i] = OUT == kOutAcc32 ? 0.f : p.scale[row0 + kRowStride * (4 * ln.kq + i)];
    bi[i] = OUT == kOutAcc32 ? 0.f : p.bias[row0 + kRowStride * (4 * ln.kq + i)];
  }
  // row n of the tile (results of the swapped product)
  const float sct = OUT == kOutAcc32 ? 0.f : p.scale[row0 + kRowStride * ln.n];
  const float bit = OUT == kOutAcc32 ? 0.f : p.bias[row0 + kRowStride * ln.n];
  __syncthreads();

  // windows shifted left by sh quads so that fp32 / int32 row pieces start on 128-byte boundaries: output row
  // r starts r * qpi quads into the tensor
  const int sh = p.align ? ((row0 * (pitch >> 2) + slab * qpi) & (kRowStride - 1)) : 0;
  const int nqt = (qpi + sh) >> 4;       // full windows
  const int left = qpi + sh - 16 * nqt;  // quads after the last window
  const int ntail = (left + 3) >> 2;
  constexpr int kElem = (OUT == kOutI8 || OUT == kOutPlanes) ? 1 : 4;
  // kOutPlanes: the wavefront's planes behind the image's cells, 16 bytes of slack in front of them
  char* planes = reinterpret_cast<char*>(lds_raw) + 256 + (size_t)NKG * kgs * 16 + wave * kPlaneBufBytes;
  char* orow = OUT == kOutPlanes ? planes + 16 : Uniform(static_cast<char*>(p.out) + (((size_t)n * p.M + row0) * pitch + slab * hw) * kElem);
  DispatchAct(OUT == kOutAcc32 ? 0 : epilogue::LeakyAsMax(p.act), [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    if (nqt > 0) {
      // wavefront w starts with window w mod nqt and goes round from there
      auto win = [&](int t) { return (t + wave) % nqt; };
      // the first line of window 0 holds the end of the previous output row when the window is shifted
      auto partial = [&](int t) { return win(t) == 0 && sh > 0; };
      v4i acc_a[4], acc_b[4];
      Window<KS, OUT, ACT, false>(xt, kgs, cps, 16 * win(0) - sh, a, acc_a, acc_a, 0, false, sc, bi, p.act, orow, pitch, ln);
      int t = 1;
      // two windows per round so that the accumulator sets alternate without copies
      for (; t + 1 < nqt; t += 2) {
        Window<KS, OUT, ACT, true>(xt, kgs, cps, 16 * win(t) - sh, a, acc_b, acc_a, 16 * win(t - 1) - sh, partial(t - 1), sc, bi, p.act, orow, pitch, ln);
        Window<KS, OUT, ACT, true>(xt, kgs, cps, 16 * win(t + 1) - sh, a, acc_a, acc_b, 16 * win(t) - sh, partial(t), sc, bi, p.act, orow, pitch, ln);
      }
      if (t < nqt) {
        Window<KS, OUT, ACT, true>(xt, kgs, cps, 16 * win(t) - sh, a, acc_b, acc_a, 16 * win(t - 1) - sh, partial(t - 1), sc, bi, p.act, orow, pitch, ln);
#pragma unroll
        for (int i = 0; i < 4; ++i) StoreRow<OUT, ACT>(acc_b, i, sc[i], bi[i], p.act, orow, pitch, 16 * win(t) - sh + ln.n, partial(t) && ln.n < kRowStride, ln);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) StoreRow<OUT, ACT>(acc_a, i, sc[i], bi[i], p.act, orow, pitch, 16 * win(t - 1) - sh + ln.n, partial(t - 1) && ln.n < kRowStride, ln);
      }
    }
    // The quads the windows leave over, four at a time, operands swapped: rows of the product are positions
    // (quad q0 + m / 4, position m % 4), columns are output rows; a lane ends with the four positions of quad
    // q0 + kq of row n.  Their lines are shared with the start of the next output row: plain stores.
    for (int t = 0; t < ntail; ++t) {
      const int q0 = 16 * nqt - sh + 4 * t;
      int tq = q0 + (ln.n >> 2);
      if (tq > qpi - 1) tq = qpi - 1;  // rows past the end of the image row: any valid cell, results unused
      if (tq < 0) tq = 0;              // likewise in front of it (rows shorter than a window, shifted left)
      const uint4* tb = xt + ln.kq * kgs + (ln.n & 3) * cps + tq;
      v4i acc = v4i{0, 0, 0, 0};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const uint4 u = tb[ks * 4 * kgs];
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)u.x, (int)u.y, (int)u.z, (int)u.w}, a[ks], acc, 0, 0, 0);
      }
      const int q = q0 + ln.kq;
      if (q >= 0 && q < qpi) {
        const u4 v = Finish4<OUT, ACT>(acc[0], acc[1], acc[2], acc[3], sct, bit, p.act);
        char* ptr = orow + ((size_t)(kPlaneStride<OUT> * ln.n) * pitch + 4 * q) * kElem;
        if (OUT == kOutPlanes) StoreLds(v.x, ptr); else if (OUT == kOutI8) StorePlain(v.x, ptr); else StorePlain(v, ptr);
      }
    }
  });
  if constexpr (OUT == kOutPlanes) DwStage<DW_STRIDE>(*dw, planes + 16, planes + kPlaneInBytes, n, p.M, row0, lane);
}

template <int KS, int OUT, int QPI, bool SLAB = false>
__global__ void __launch_bounds__(512) ImageRowsMfmaKernel(PL_HEAD_PARAMS, const ImageMfmaParams block) {
  const ImageMfmaParams p = WithHead(block, PL_HEAD_ARGS);
  extern __shared__ uint4 lds_raw[];
  RowsBody<KS, OUT, QPI, 0, SLAB>(p, lds_raw, nullptr);
}

// The same followed by the depthwise 3 x 3 layer (14 x 14 planes, padding 1, stride DW_STRIDE, int8 output) on
// the wavefront's own 16 planes: the pointwise output never leaves the CU.
template <int KS, int DW_STRIDE>
__global__ void __launch_bounds__(512) ImageRowsDwKernel(PL_HEAD_PARAMS, const ImageMfmaParams block, const DwConvParams dw) {
  const ImageMfmaParams p = WithHead(block, PL_HEAD_ARGS);
  extern __shared__ uint4 lds_raw[];
  RowsBody<KS, kOutPlanes, 49, DW_STRIDE>(p, lds_raw, &dw);
}

template <int OUT>
hipError_t ByKs(const ImageMfmaParams& q, dim3 grid, size_t lds, hipStream_t s) {
  const dim3 block(512);
  if (q.slabs > 1) {  // slabs of 196 positions
    switch (q.K / 64) {
      case 2:
        return LaunchWithHead(ImageRowsMfmaKernel<2, OUT, 49, true>, grid, block, lds, s, q);
      case 4:
        return LaunchWithHead(ImageRowsMfmaKernel<4, OUT, 49, true>, grid, block, lds, s, q);
      case 8:
        return LaunchWithHead(ImageRowsMfmaKernel<8, OUT, 49, true>, grid, block, lds, s, q);
      default:
        return hipErrorInvalidValue;
    }
  }
  if (q.qpi == 49) {
    switch (q.K / 64) {
      case 2:
        return LaunchWithHead(ImageRowsMfmaKernel<2, OUT, 49>, grid, block, lds, s, q);
      case 4:
        return LaunchWithHead(ImageRowsMfmaKernel<4, OUT, 49>, grid, block, lds, s, q);
      case 8:
        return LaunchWithHead(ImageRowsMfmaKernel<8, OUT, 49>, grid, block, lds, s, q);
      default:
        return hipErrorInvalidValue;
    }
  }
  switch (q.K / 64) {
    case 2:
      return LaunchWithHead(ImageRowsMfmaKernel<2, OUT, 0>, grid, block, lds, s, q);
    case 4:
      return LaunchWithHead(ImageRowsMfmaKernel<4, OUT, 0>, grid, block, lds, s, q);
    case 8:
      return LaunchWithHead(ImageRowsMfmaKernel<8, OUT, 0>, grid, block, lds, s, q);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace

bool ImageRowsMfmaFits(int M, int K, int hw) {
  if (M <= 0 || M % 128 != 0) return false;
  if (K != 128 && K != 256 && K != 512) return false;
  if (hw < 16 || hw > 256 || hw % 4 != 0) return false;
  const int qpi = hw / 4, kgs = (4 * qpi + 15) / 16 * 16;
  return 256 + (size_t)(K / 16) * kgs * 16 <= (size_t)kMaxLdsBytes;
}

constexpr int kSlab = 196;  // positions of a slab of a larger map (49 quads: the kernel's compile-time row length)

bool ImageRowsSlabFits(int M, int K, int hw) { return hw > 256 && hw % kSlab == 0 && ImageRowsMfmaFits(M, K, kSlab); }

// p.hw: positions of the whole map; it is taken whole where it fits, else in slabs of 196 positions.
hipError_t LaunchImageRowsMfma(int out_kind, const ImageMfmaParams& p, hipStream_t stream) {
  if (p.batch <= 0) return hipSuccess;
  const bool whole = ImageRowsMfmaFits(p.M, p.K, p.hw);
  if (!whole && !ImageRowsSlabFits(p.M, p.K, p.hw)) return hipErrorInvalidValue;
  // the image is read as dwords, the output written as 16-byte pieces
  if (reinterpret_cast<uintptr_t>(p.x) % 4 != 0 || reinterpret_cast<uintptr_t>(p.out) % 16 != 0) return hipErrorInvalidValue;
  ImageMfmaParams q = p;
  q.pitch = p.hw;
  q.slabs = whole ? 1 : p.hw / kSlab;
  q.hw = whole ? p.hw : kSlab;
  q.qpi = q.hw / 4;
  q.kgs = (4 * q.qpi + 15) / 16 * 16;  // a channel group's cells start on a 256-byte boundary: conflict-free operand reads
  q.row_groups = p.M / 128;
  if ((int64_t)p.batch * p.K * p.hw >= (1ll << 40)) return hipErrorInvalidValue;
  const int64_t items = (int64_t)p.batch * q.slabs * q.row_groups;
  if (items > (1 << 28)) return hipErrorInvalidValue;
  q.items = (int)items;
  q.per_xcd = (q.items + 7) / 8;
  q.align = out_kind != kOutI8;
  const size_t lds = 256 + (size_t)(p.K / 16) * q.kgs * 16;
  const dim3 grid(8u * (uint32_t)q.per_xcd);
  switch (out_kind) {
    case kOutF32:
      return ByKs<kOutF32>(q, grid, lds, stream);
    case kOutI8:
      return ByKs<kOutI8>(q, grid, lds, stream);
    case kOutAcc32:
      return ByKs<kOutAcc32>(q, grid, lds, stream);
    default:
      return hipErrorInvalidValue;
  }
}

// The pointwise layer followed by the depthwise 3 x 3 layer on its output, in one launch (14 x 14 maps).
bool ImageRowsDwFits(int M, int K, int hw, int h, int w, int pad, int stride) {
  if (!ImageRowsMfmaFits(M, K, hw) || hw != 196 || h != 14 || w != 14 || pad != 1 || (stride != 1 && stride != 2)) return false;
  return 256 + (size_t)(K / 16) * 208 * 16 + (size_t)8 * kPlaneBufBytes <= (size_t)kMaxLdsBytes;
}

hipError_t LaunchImageRowsDw(const ImageMfmaParams& p, const DwConvParams& d, int stride, hipStream_t stream) {
  if (p.batch <= 0) return hipSuccess;
  if (!ImageRowsDwFits(p.M, p.K, p.hw, d.h, d.w, d.pad, stride) || d.channels != p.M) return hipErrorInvalidValue;
  const int oh = (14 + 2 - 3) / stride + 1;
  if (d.oh != oh || d.ow != oh) return hipErrorInvalidValue;
  // the image is read as dwords; planes of 196 bytes are stored as dwords, planes of 49 bytes byte by byte
  if (reinterpret_cast<uintptr_t>(p.x) % 4 != 0 || (stride == 1 && reinterpret_cast<uintptr_t>(d.out) % 4 != 0)) return hipErrorInvalidValue;
  ImageMfmaParams q = p;
  q.pitch = p.hw;
  q.slabs = 1;
  q.qpi = 49;
  q.kgs = 208;
  q.row_groups = p.M / 128;
  const int64_t items = (int64_t)p.batch * q.row_groups;
  if (items > (1 << 28)) return hipErrorInvalidValue;
  q.items = (int)items;
  q.per_xcd = (q.items + 7) / 8;
  q.align = 0;
  const size_t lds = 256 + (size_t)(p.K / 16) * q.kgs * 16 + (size_t)8 * kPlaneBufBytes;
  const dim3 grid(8u * (uint32_t)q.per_xcd), block(512);
  const int shape = 10 * (p.K / 64) + stride;
  switch (shape) {
    case 21:
      return LaunchWithHead(ImageRowsDwKernel<2, 1>, grid, block, lds, stream, q, d);
    case 22:
      return LaunchWithHead(ImageRowsDwKernel<2, 2>, grid, block, lds, stream, q, d);
    case 41:
      return LaunchWithHead(ImageRowsDwKernel<4, 1>, grid, block, lds, stream, q, d);
    case 42:
      return LaunchWithHead(ImageRowsDwKernel<4, 2>, grid, block, lds, stream, q, d);
    case 81:
      return LaunchWithHead(ImageRowsDwKernel<8, 1>, grid, block, lds, stream, q, d);
    case 82:
      return LaunchWithHead(ImageRowsDwKernel<8, 2>, grid, block, lds, stream, q, d);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace pl
