// Image MFMA: int8 sparse 1x1 convolution for feature maps small enough that
// one image's activations ([K x H*W] int8, at most 128 KB) fit the LDS of a CU.
//
// One workgroup of eight wavefronts computes 128 output rows of one image.
//   * The image is brought in once as whole cache lines: every wavefront
//     moves its channel groups (16 channels x H*W bytes, contiguous in NCHW)
//     from global memory straight into LDS (global_load_lds, no registers),
//     then turns each group in place into matrix-core operand cells
//     (16 channels of one position = 16 bytes) with 4x4 byte transposes.
//   * Weights are dense 16x64 int8 tiles in v_mfma_i32_16x16x64_i8 operand
//     order, held in registers (a wavefront pair shares 32 rows).  The rows of
//     a tile are rho, rho + 4, rho + 8, ...: all rows of a tile then start at
//     the same offset inside a 64-byte sector of the fp32 output, and the
//     tile's window of 16 position quads is shifted left by that offset so
//     that every 256-byte row piece it stores covers whole sectors.  Those
//     are written through to memory (sc1 nt); the few pieces that share a
//     sector with a neighbouring row are stored plainly and merge in L2.
//   * The channel loop is innermost: a window is finished and stored while
//     the other wavefront of the SIMD multiplies, so stores start right after
//     the first window instead of after the whole tile.
//   * The quads that the shifted windows leave over at the end of a row are
//     computed with the operands swapped (positions as matrix rows).
// A second kernel below takes 7 x 7 maps, two images per workgroup.
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

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
// the same with the alignment of its elements only: rows of 49 outputs start anywhere
typedef uint32_t u4a __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u1a __attribute__((aligned(1)));

// 16 bytes written through to memory as streaming data (sc1 nt).  Measured on
// 64 x 512 -> 512 @14x14, fp32 output, whole sectors: plain 13.8 us, sc1 12.3,
// nt 11.1, sc1 nt 10.8.  The wait state after the store keeps the data
// registers intact until the store has read them (the compiler does not see a
// store inside the assembly statement).
__device__ __forceinline__ void StoreThrough(u4 v, void* p) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n s_nop 1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void StorePlain(u4 v, void* p) { *reinterpret_cast<u4*>(p) = v; }

struct Lane {
  int n;   // column of a 16x16 tile
  int kq;  // quarter of the wavefront: channel group of an operand, rows 4 kq .. 4 kq + 3 of a result
};

// Per-wavefront constants of the epilogue.
struct Rows {
  float sc[2][4], bi[2][4];  // rows 4 kq + i of the wavefront's two row tiles
  float sct[2], bit[2];      // row n of each tile (results of the swapped product)
};

// Epilogue of four accumulators (positions 4 q .. 4 q + 3 of one output row).
template <int OUT, int ACT>
__device__ __forceinline__ u4 Finish4(int a0, int a1, int a2, int a3, float s, float b, const DevAct& act) {
  if (OUT == kOutAcc32) return u4{(uint32_t)a0, (uint32_t)a1, (uint32_t)a2, (uint32_t)a3};
  const float v0 = __builtin_fmaf((float)a0, s, b), v1 = __builtin_fmaf((float)a1, s, b), v2 = __builtin_fmaf((float)a2, s, b), v3 = __builtin_fmaf((float)a3, s, b);
  if (OUT == kOutI8) return u4{TruncPackI8x4(ActQuantF<ACT>(v0, act), ActQuantF<ACT>(v1, act), ActQuantF<ACT>(v2, act), ActQuantF<ACT>(v3, act)), 0u, 0u, 0u};
  return u4{__float_as_uint(ActivateT<ACT>(v0, act)), __float_as_uint(ActivateT<ACT>(v1, act)), __float_as_uint(ActivateT<ACT>(v2, act)), __float_as_uint(ActivateT<ACT>(v3, act))};
}

// One window of 16 position quads times NOC row tiles (tiles J0 .. J0 + NOC - 1
// of the wavefront): 4 * NOC matrix instructions per k-step, then the stores.
//   q0: first quad of the window (may be negative: the quads in front of the
//       row belong to the previous row and are not stored)
//   orow: output row of MFMA row 0 of tile 0, element units of the output type
template <int KS, int OUT, int NOC, int J0>
__device__ __forceinline__ void Window(const uint4* __restrict__ xt, int kgs, int qpi, int q0, bool first_sector_shared, const v4i (&a)[2][KS], const Rows& rw, const DevAct& act, char* __restrict__ orow, int hw,
                                       Lane ln) {
  const int q = q0 + ln.n;
  const uint4* bbase = xt + ln.kq * kgs + q;  // + ks * 4 * kgs + c * qpi
  v4i acc[NOC][4];
#pragma unroll
  for (int o = 0; o < NOC; ++o)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[o][c] = v4i{0, 0, 0, 0};
  uint4 bq[2][4];
#pragma unroll
  for (int c = 0; c < 4; ++c) bq[0][c] = bbase[c * qpi];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (ks + 1 < KS) {
#pragma unroll
      for (int c = 0; c < 4; ++c) bq[(ks + 1) & 1][c] = bbase[(ks + 1) * 4 * kgs + c * qpi];
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint4 u = bq[ks & 1][c];
      const v4i bv = v4i{(int)u.x, (int)u.y, (int)u.z, (int)u.w};
#pragma unroll
      for (int o = 0; o < NOC; ++o) acc[o][c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[J0 + o][ks], bv, acc[o][c], 0, 0, 0);
    }
  }
  constexpr int kElem = OUT == kOutI8 ? 1 : 4;
  // the first sector of a shifted window is shared with the end of the previous row
  const bool shared = first_sector_shared && ln.n < 4;
  DispatchAct(OUT == kOutAcc32 ? 0 : act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int o = 0; o < NOC; ++o) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u4 v = Finish4<OUT, ACT>(acc[o][0][i], acc[o][1][i], acc[o][2][i], acc[o][3][i], rw.sc[J0 + o][i], rw.bi[J0 + o][i], act);
        // rows of a tile are 4 apart: MFMA row m of tile j is row 4 (16 j + m) past the wavefront's first row
        char* ptr = orow + ((size_t)(4 * (16 * (J0 + o) + 4 * ln.kq + i)) * hw + 4 * q) * kElem;
        if (OUT == kOutI8) {
          if (q >= 0) *reinterpret_cast<uint32_t*>(ptr) = v.x;
        } else if (shared) {
          if (q >= 0) StorePlain(v, ptr);
        } else {
          StoreThrough(v, ptr);
        }
      }
    }
  });
}

// Four quads starting at quad q0, both row tiles, operands swapped: rows of
// the product are positions (quad q0 + m / 4, position m % 4), columns are
// output rows.  A lane ends with the four positions of quad q0 + kq of row n.
template <int KS, int OUT>
__device__ __forceinline__ void Tail(const uint4* __restrict__ xt, int kgs, int qpi, int q0, const v4i (&a)[2][KS], const Rows& rw, const DevAct& act, char* __restrict__ orow, int hw, Lane ln) {
  int tq = q0 + (ln.n >> 2);
  if (tq > qpi - 1) tq = qpi - 1;  // rows past the end of the image row: any valid cell, results unused
  if (tq < 0) tq = 0;              // likewise in front of it (rows shorter than a window, shifted left)
  const uint4* tb = xt + ln.kq * kgs + (ln.n & 3) * qpi + tq;
  v4i acc[2] = {v4i{0, 0, 0, 0}, v4i{0, 0, 0, 0}};
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const uint4 u = tb[ks * 4 * kgs];
    const v4i av = v4i{(int)u.x, (int)u.y, (int)u.z, (int)u.w};
#pragma unroll
    for (int o = 0; o < 2; ++o) acc[o] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, a[o][ks], acc[o], 0, 0, 0);
  }
  constexpr int kElem = OUT == kOutI8 ? 1 : 4;
  const int q = q0 + ln.kq;
  // quads in front of the row belong to the previous row's last sector and are written by its wavefront
  if (q < 0 || q >= qpi) return;
  DispatchAct(OUT == kOutAcc32 ? 0 : act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int o = 0; o < 2; ++o) {
      const u4 v = Finish4<OUT, ACT>(acc[o][0], acc[o][1], acc[o][2], acc[o][3], rw.sct[o], rw.bit[o], act);
      char* ptr = orow + ((size_t)(4 * (16 * o + ln.n)) * hw + 4 * q) * kElem;
      if (OUT == kOutI8) *reinterpret_cast<uint32_t*>(ptr) = v.x; else StorePlain(v, ptr);
    }
  });
}

// QPI: quads per image when known at compile time (49 = 14 x 14 maps), else 0.
// With the constant, the LDS offsets of the regrouping and of the operand
// reads become immediates (64 x 512 -> 512 @14x14: 10.8 -> 10.4 us); the image
// size in bytes stays a run-time value on purpose (as a constant it changed the
// schedule of the direct loads and the stores and cost more than it saved).
//
// TRG (512 channels, 14 x 14 maps): the regrouping is done by the LDS itself.  ds_read_b64_tr_b8 hands
// lane j of a group of 16 lanes byte j % 8 of the eight bytes that lane 2 b + j / 8 of the group addressed, as
// its byte b: eight channels of one position per lane when the 16 lanes address eight channel rows (two
// runs of eight positions each).  Two such reads are one operand cell, which is then written where the
// windows expect it; no vector ALU transposes (64 x 512 -> 512 @14x14: 9.7 -> see the measurements).  The
// read ignores the low three address bits and rows of 196 bytes start 8-byte aligned only for even
// channels, so a cell holds channels of one parity (for odd channels the aligned runs cover positions
// 8 u + 4 .. 8 u + 11), and channels of a cell are four apart so that the 16 rows of a half wavefront fall
// into different banks: channel 64 ks + 4 (8 (g % 2) + b % 8) + 2 (b / 8) + g / 2 is byte b of cell group g
// of k-step ks.  The weight tiles come in the same order (the order inside an integer dot product is free).
template <int KS, int OUT, int QPI, bool TRG = false>
__global__ void __launch_bounds__(512) ImageMfmaKernel(PL_HEAD_PARAMS, const ImageMfmaParams block) {
  const ImageMfmaParams p = WithHead(block, PL_HEAD_ARGS);
  extern __shared__ uint4 lds_raw[];
  // shifted windows read up to three cells in front of a row of cells
  uint4* xt = lds_raw + 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // a contiguous range of work items per XCD, the row groups of one image next to each other
  const int item = (int)(blockIdx.x & 7u) * p.per_xcd + (int)(blockIdx.x >> 3);
  if (item >= p.items) return;
  const int n = item / p.row_groups, rg = item - n * p.row_groups;
  const int rho = wave & 3, half = wave >> 2;
  const int qpi = QPI ? QPI : p.qpi, kgs = QPI ? (4 * QPI + 15) / 16 * 16 : p.kgs, hw = p.hw;
  constexpr int NKG = 4 * KS, BPW = NKG / 8;
  static_assert(NKG % 8 == 0, "channel groups are dealt evenly to the eight wavefronts");

  // activations: channel groups straight into LDS, whole lines
  const int8_t* ximg = p.x + (size_t)n * p.K * hw;
  char* lbase = reinterpret_cast<char*>(xt);
  const int blk_bytes = 16 * hw;
  if (TRG) {
    // the wavefront's 64 channel rows as they lie in memory, at the start of the region of its four cell groups
    const int bytes = BPW * blk_bytes;
    const int8_t* src = ximg + (size_t)wave * bytes + lane * 16;
    char* dst = lbase + wave * BPW * (kgs * 16);
    const int full = bytes >> 10, rem_lanes = (bytes & 1023) >> 4;
    for (int t = 0; t < full; ++t)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + t * 1024), (__attribute__((address_space(3))) void*)(dst + t * 1024), 16, 0, 0);
    if (lane < rem_lanes)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + full * 1024), (__attribute__((address_space(3))) void*)(dst + full * 1024), 16, 0, 0);
  } else {
#pragma unroll
    for (int u = 0; u < BPW; ++u) {
      const int kg = wave * BPW + u;
      const int8_t* src = ximg + (size_t)kg * blk_bytes + lane * 16;
      char* dst = lbase + kg * (kgs * 16);
      for (int t = 0; t < p.dma_full; ++t)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + t * 1024), (__attribute__((address_space(3))) void*)(dst + t * 1024), 16, 0, 0);
      if (lane < p.dma_rem_lanes)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + p.dma_full * 1024), (__attribute__((address_space(3))) void*)(dst + p.dma_full * 1024), 16, 0, 0);
    }
  }
  // Every channel group of this wavefront has landed.  (The builtin, not an assembly statement: the
  // compiler then knows that no direct load is in flight any more and puts no wait of its own in front
  // of the LDS accesses below.)
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  // The weights, scales and biases are requested now and arrive while the activations are regrouped:
  // LDS operations wait for direct loads that may still be in flight, not for ordinary ones.
  // weights of the wavefront's two row tiles, all channels
  v4i a[2][KS];
  const v4i* wt = static_cast<const v4i*>(p.wtiles) + ((size_t)(rg * 4 + rho) * 2 * KS) * 64 + lane;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) a[j][ks] = wt[(j * KS + ks) * 64];
  Lane ln;
  ln.n = lane & 15;
  ln.kq = lane >> 4;
  const int row0 = rg * 128 + rho;  // the wavefront's rows: row0 + 4 m, m = 0 .. 31
  Rows rw;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      rw.sc[j][i] = OUT == kOutAcc32 ? 0.f : p.scale[row0 + 4 * (16 * j + 4 * ln.kq + i)];
      rw.bi[j][i] = OUT == kOutAcc32 ? 0.f : p.bias[row0 + 4 * (16 * j + 4 * ln.kq + i)];
    }
    rw.sct[j] = OUT == kOutAcc32 ? 0.f : p.scale[row0 + 4 * (16 * j + ln.n)];
    rw.bit[j] = OUT == kOutAcc32 ? 0.f : p.bias[row0 + 4 * (16 * j + ln.n)];
  }
  if (TRG) {
    static_assert(!TRG || (KS == 8 && QPI > 0 && (QPI & 1)), "regrouping by transposing reads: 512 channels, rows of 4 (mod 8) bytes");
    typedef int v2i __attribute__((ext_vector_type(2)));
    auto reg = (__attribute__((address_space(3))) char*)lbase + wave * BPW * (kgs * 16);
    const int g = lane >> 4, s16 = lane & 15, par = g >> 1;
    // the lane addresses channel row 4 (8 (g % 2) + s16 / 2) + g / 2 (+ 2 for the second read), run s16 % 2
    const int rbase = (4 * (8 * (g & 1) + (s16 >> 1)) + par) * hw + 8 * (s16 & 1) - 4 * par;
    constexpr int NWIN = (4 * QPI + 3) / 16 + 1;  // windows of 16 positions; those of odd channels start at -4
    v2i rr[NWIN][2];
#pragma unroll
    for (int i = 0; i < NWIN; ++i)
#pragma unroll
      for (int r2 = 0; r2 < 2; ++r2) rr[i][r2] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<__attribute__((address_space(3))) v2i*>(reg + rbase + 16 * i + 2 * r2 * hw));
    // every lane has read before any lane overwrites
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_sched_barrier(0);
    auto cells = reinterpret_cast<__attribute__((address_space(3))) v4i*>(reg + g * (kgs * 16));
#pragma unroll
    for (int i = 0; i < NWIN; ++i) {
      const int pos = 16 * i - 4 * par + s16;
      if (pos >= 0 && pos < 4 * QPI) cells[(pos & 3) * QPI + (pos >> 2)] = v4i{rr[i][0].x, rr[i][0].y, rr[i][1].x, rr[i][1].y};
    }
  } else {
  // in place: 16 dwords (16 channels x 4 positions) per quad -> 4 cells.  The dwords of all of the
  // wavefront's channel groups are read first (one wait instead of one per group), then every group is
  // transposed and written back; a group is touched by this wavefront only.
  uint32_t r[BPW][16];
  if (lane < qpi) {
#pragma unroll
    for (int u = 0; u < BPW; ++u) {
      const uint32_t* blk = reinterpret_cast<const uint32_t*>(lbase + (wave * BPW + u) * (kgs * 16));
#pragma unroll
      for (int i = 0; i < 16; ++i) r[u][i] = blk[i * qpi + lane];
    }
  }
  // every lane has read before any lane overwrites
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_sched_barrier(0);
  if (lane < qpi) {
#pragma unroll
    for (int u = 0; u < BPW; ++u) {
      // Two stages of byte permutes.  The second stage is done cell by cell so
      // that the four dwords of a cell (one per block of four channels) are
      // produced next to each other, where the 16-byte store wants them.
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
  }
  }
  __syncthreads();

  // windows: shifted left by sh quads so that fp32 / int32 row pieces start on 64-byte boundaries
  const int sh = p.align ? ((rho * qpi) & 3) : 0;
  const int nqt = (qpi + sh) >> 4;            // full windows
  const int left = qpi + sh - 16 * nqt;       // quads after the last window
  const int ntail = (left + 3) >> 2;
  // split between the two wavefronts of the pair, in matrix instructions per k-step:
  // window x both tiles = 8, window x one tile = 4, tail = 2
  const int target = (8 * nqt + 2 * ntail) >> 1;
  const int wa = target >> 3;
  const bool split = (target - 8 * wa) >= 2 && wa < nqt;
  constexpr int kElem = OUT == kOutI8 ? 1 : 4;
  char* orow = static_cast<char*>(p.out) + ((size_t)n * p.M + row0) * hw * kElem;
  if (half == 0) {
    if (split) Window<KS, OUT, 1, 0>(xt, kgs, qpi, 16 * wa - sh, wa == 0 && sh > 0, a, rw, p.act, orow, hw, ln);
    for (int T = 0; T < wa; ++T) Window<KS, OUT, 2, 0>(xt, kgs, qpi, 16 * T - sh, T == 0 && sh > 0, a, rw, p.act, orow, hw, ln);
  } else {
    const int first = wa + (split ? 1 : 0);
    for (int T = nqt - 1; T >= first; --T) Window<KS, OUT, 2, 0>(xt, kgs, qpi, 16 * T - sh, T == 0 && sh > 0, a, rw, p.act, orow, hw, ln);
    if (split) Window<KS, OUT, 1, 1>(xt, kgs, qpi, 16 * wa - sh, wa == 0 && sh > 0, a, rw, p.act, orow, hw, ln);
    for (int t = 0; t < ntail; ++t) Tail<KS, OUT>(xt, kgs, qpi, 16 * nqt - sh + 4 * t, a, rw, p.act, orow, hw, ln);
  }
}

// ---------------------------------------------------------------------------
// 7 x 7 maps.  A channel row is 49 bytes, so rows are not dword aligned and an
// image is small: a workgroup takes two images (98 positions) and 128 output
// rows.  A unit is one channel group of one image (16 x 49 = 784 bytes,
// contiguous in NCHW, a multiple of 16): it is moved into LDS by 49 lanes of
// one direct load, into a slot of 1 KB, and regrouped in place there into 13
// quads x 4 cells (the last quad holds position 48 and three bytes that are
// never used).  Lanes regroup four units at a time (13 quads each); a
// channel's dword of a quad is put together from the two aligned dwords it
// straddles (v_alignbyte_b32, shift = channel mod 4).
// The 26 quads of the two images form two windows of 16 quad columns, one per
// wavefront of a pair; a lane's column is (image, quad) = (g / 13, g % 13).
constexpr int kSmallHw = 49, kSmallQuads = 13, kSmallSlotCells = 64;

template <int KS, int OUT>
__global__ void __launch_bounds__(512) SmallMapMfmaKernel(PL_HEAD_PARAMS, const ImageMfmaParams block) {
  const ImageMfmaParams p = WithHead(block, PL_HEAD_ARGS);
  extern __shared__ uint4 lds_raw[];
  uint4* xt = lds_raw + 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int item = (int)(blockIdx.x & 7u) * p.per_xcd + (int)(blockIdx.x >> 3);
  if (item >= p.items) return;
  const int pair = item / p.row_groups, rg = item - pair * p.row_groups;
  const int n0 = 2 * pair;
  const int n_img = min(2, p.batch - n0);  // the last pair of an odd batch holds one image
  const int rho = wave & 3, half = wave >> 2;
  constexpr int NKG = 4 * KS, UNITS = 2 * NKG, UPW = UNITS / 8;
  static_assert(UPW % 4 == 0, "units are regrouped four at a time");
  constexpr int kSlotBytes = kSmallSlotCells * 16;

  // activations: one direct load per unit, 49 lanes x 16 bytes
  char* lbase = reinterpret_cast<char*>(xt);
#pragma unroll
  for (int t = 0; t < UPW; ++t) {
    const int u = wave * UPW + t;
    const int m = u / NKG, kg = u % NKG;
    const int img = n0 + min(m, n_img - 1);  // a missing second image repeats the first; its results are not stored
    const int8_t* src = p.x + ((size_t)img * p.K + 16 * kg) * kSmallHw + lane * 16;
    if (lane < kSmallHw) __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src, (__attribute__((address_space(3))) void*)(lbase + u * kSlotBytes), 16, 0, 0);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the builtin, so that the compiler knows no direct load is in flight
  // weights of the wavefront's two row tiles (all channels), scales and biases: they arrive during the regrouping
  v4i a[2][KS];
  const v4i* wt = static_cast<const v4i*>(p.wtiles) + ((size_t)(rg * 4 + rho) * 2 * KS) * 64 + lane;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) a[j][ks] = wt[(j * KS + ks) * 64];
  Lane ln;
  ln.n = lane & 15;
  ln.kq = lane >> 4;
  const int row0 = rg * 128 + rho;  // the wavefront's rows: row0 + 4 m, m = 0 .. 31
  Rows rw;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      rw.sc[j][i] = OUT == kOutAcc32 ? 0.f : p.scale[row0 + 4 * (16 * j + 4 * ln.kq + i)];
      rw.bi[j][i] = OUT == kOutAcc32 ? 0.f : p.bias[row0 + 4 * (16 * j + 4 * ln.kq + i)];
    }
    rw.sct[j] = rw.bit[j] = 0.f;
  }

  // regrouping in place, four units per pass: lane = 13 * (unit of the pass) + quad
  {
    const int uj = (lane * 20) >> 8;  // lane / 13 for lane < 64
    const int q = lane - kSmallQuads * uj;
#pragma unroll
    for (int pass = 0; pass < UPW / 4; ++pass) {
      char* slot = lbase + (wave * UPW + 4 * pass + uj) * kSlotBytes;
      const uint32_t* words = reinterpret_cast<const uint32_t*>(slot) + q;
      uint32_t r[16];
      if (lane < 4 * kSmallQuads) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          // bytes 49 i + 4 q .. + 3 of the unit: dword (49 i >> 2) + q, shifted by i mod 4 bytes
          const uint32_t d0 = words[(kSmallHw * i) >> 2];
          if ((i & 3) == 0) {
            r[i] = d0;
          } else {
            const uint32_t d1 = words[((kSmallHw * i) >> 2) + 1];
            r[i] = __builtin_amdgcn_alignbyte(d1, d0, i & 3);
          }
        }
      }
      // every lane has read before any lane overwrites
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_sched_barrier(0);
      if (lane < 4 * kSmallQuads) {
        uint32_t lo[4][2], hi[4][2];
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          lo[b4][0] = __builtin_amdgcn_perm(r[4 * b4 + 1], r[4 * b4], 0x05010400u);
          hi[b4][0] = __builtin_amdgcn_perm(r[4 * b4 + 1], r[4 * b4], 0x07030602u);
          lo[b4][1] = __builtin_amdgcn_perm(r[4 * b4 + 3], r[4 * b4 + 2], 0x05010400u);
          hi[b4][1] = __builtin_amdgcn_perm(r[4 * b4 + 3], r[4 * b4 + 2], 0x07030602u);
        }
        uint4* cells = reinterpret_cast<uint4*>(slot) + q;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
          uint4 cell;
          cell.x = __builtin_amdgcn_perm((c & 2) ? hi[0][1] : lo[0][1], (c & 2) ? hi[0][0] : lo[0][0], sel);
          cell.y = __builtin_amdgcn_perm((c & 2) ? hi[1][1] : lo[1][1], (c & 2) ? hi[1][0] : lo[1][0], sel);
          cell.z = __builtin_amdgcn_perm((c & 2) ? hi[2][1] : lo[2][1], (c & 2) ? hi[2][0] : lo[2][0], sel);
          cell.w = __builtin_amdgcn_perm((c & 2) ? hi[3][1] : lo[3][1], (c & 2) ? hi[3][0] : lo[3][0], sel);
          cells[c * kSmallQuads] = cell;
        }
      }
    }
  }
  __syncthreads();

  // the wavefront's window: quad columns 16 half .. 16 half + 15 of the 26
  const int g = 16 * half + ln.n;
  const bool live = g < 2 * kSmallQuads;
  const int gc = live ? g : 2 * kSmallQuads - 1;
  const int m = gc >= kSmallQuads ? 1 : 0, ql = gc - kSmallQuads * m;
  const uint4* bbase = xt + (m * NKG + ln.kq) * kSmallSlotCells + ql;  // + ks * 4 * kSmallSlotCells + c * kSmallQuads
  v4i acc[2][4];
#pragma unroll
  for (int o = 0; o < 2; ++o)
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[o][c] = v4i{0, 0, 0, 0};
  uint4 bq[2][4];
#pragma unroll
  for (int c = 0; c < 4; ++c) bq[0][c] = bbase[c * kSmallQuads];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (ks + 1 < KS) {
#pragma unroll
      for (int c = 0; c < 4; ++c) bq[(ks + 1) & 1][c] = bbase[(ks + 1) * 4 * kSmallSlotCells + c * kSmallQuads];
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint4 u = bq[ks & 1][c];
      const v4i bv = v4i{(int)u.x, (int)u.y, (int)u.z, (int)u.w};
#pragma unroll
      for (int o = 0; o < 2; ++o) acc[o][c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[o][ks], bv, acc[o][c], 0, 0, 0);
    }
  }
  if (!live || m >= n_img) return;
  constexpr int kElem = OUT == kOutI8 ? 1 : 4;
  char* obase = static_cast<char*>(p.out) + (((size_t)(n0 + m) * p.M + row0) * kSmallHw + 4 * ql) * kElem;
  const bool last = ql == kSmallQuads - 1;  // position 48 only
  DispatchAct(OUT == kOutAcc32 ? 0 : p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int o = 0; o < 2; ++o) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u4 v = Finish4<OUT, ACT>(acc[o][0][i], acc[o][1][i], acc[o][2][i], acc[o][3][i], rw.sc[o][i], rw.bi[o][i], p.act);
        char* ptr = obase + (size_t)(4 * (16 * o + 4 * ln.kq + i)) * kSmallHw * kElem;
        if (OUT == kOutI8) {
          if (last) *reinterpret_cast<uint8_t*>(ptr) = (uint8_t)(v.x & 0xffu);
          else *reinterpret_cast<u1a*>(ptr) = v.x;
        } else {
          if (last) *reinterpret_cast<uint32_t*>(ptr) = v.x;
          else *reinterpret_cast<u4a*>(ptr) = v;
        }
      }
    }
  });
}

template <int OUT>
hipError_t SmallByKs(const ImageMfmaParams& q, dim3 grid, size_t lds, hipStream_t s) {
  const dim3 block(512);
  switch (q.K / 64) {
    case 4:
      return LaunchWithHead(SmallMapMfmaKernel<4, OUT>, grid, block, lds, s, q);
    case 8:
      return LaunchWithHead(SmallMapMfmaKernel<8, OUT>, grid, block, lds, s, q);
    case 16:
      return LaunchWithHead(SmallMapMfmaKernel<16, OUT>, grid, block, lds, s, q);
    default:
      return hipErrorInvalidValue;
  }
}

template <int OUT>
hipError_t ByKs(const ImageMfmaParams& q, dim3 grid, size_t lds, hipStream_t s) {
  const dim3 block(512);
  if (q.qpi == 49) {
    switch (q.K / 64) {
      case 2:
        return LaunchWithHead(ImageMfmaKernel<2, OUT, 49>, grid, block, lds, s, q);
      case 4:
        return LaunchWithHead(ImageMfmaKernel<4, OUT, 49>, grid, block, lds, s, q);
      case 8:
        if (q.tr_regroup) return LaunchWithHead(ImageMfmaKernel<8, OUT, 49, true>, grid, block, lds, s, q);
        return LaunchWithHead(ImageMfmaKernel<8, OUT, 49>, grid, block, lds, s, q);
      default:
        return hipErrorInvalidValue;
    }
  }
  switch (q.K / 64) {
    case 2:
      return LaunchWithHead(ImageMfmaKernel<2, OUT, 0>, grid, block, lds, s, q);
    case 4:
      return LaunchWithHead(ImageMfmaKernel<4, OUT, 0>, grid, block, lds, s, q);
    case 8:
      return LaunchWithHead(ImageMfmaKernel<8, OUT, 0>, grid, block, lds, s, q);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace

bool ImageMfmaFits(int M, int K, int hw) {
  if (M <= 0 || M % 128 != 0) return false;
  if (hw == kSmallHw) return (K == 256 || K == 512 || K == 1024) && 256 + (size_t)2 * (K / 16) * kSmallSlotCells * 16 <= (size_t)kMaxLdsBytes;
  if (K != 128 && K != 256 && K != 512) return false;
  if (hw < 16 || hw > 256 || hw % 4 != 0) return false;
  const int qpi = hw / 4, kgs = (4 * qpi + 15) / 16 * 16;
  return 256 + (size_t)(K / 16) * kgs * 16 <= (size_t)kMaxLdsBytes;
}

bool ImageMfmaRegroupsByTransposingReads(int K, int hw) { return K == 512 && hw == 196; }

hipError_t LaunchImageMfma(int out_kind, const ImageMfmaParams& p, hipStream_t stream) {
  if (p.batch <= 0) return hipSuccess;
  if (p.tr_regroup && !ImageMfmaRegroupsByTransposingReads(p.K, p.hw)) return hipErrorInvalidValue;
  if (!ImageMfmaFits(p.M, p.K, p.hw)) return hipErrorInvalidValue;
  if (reinterpret_cast<uintptr_t>(p.x) % 16 != 0 || reinterpret_cast<uintptr_t>(p.out) % 16 != 0) return hipErrorInvalidValue;
  ImageMfmaParams q = p;
  if (p.hw == kSmallHw) {
    q.row_groups = p.M / 128;
    const int64_t small_items = (int64_t)((p.batch + 1) / 2) * q.row_groups;
    if (small_items > (1 << 28)) return hipErrorInvalidValue;
    q.items = (int)small_items;
    q.per_xcd = (q.items + 7) / 8;
    const size_t small_lds = 256 + (size_t)2 * (p.K / 16) * kSmallSlotCells * 16;
    const dim3 small_grid(8u * (uint32_t)q.per_xcd);
    switch (out_kind) {
      case kOutF32:
        return SmallByKs<kOutF32>(q, small_grid, small_lds, stream);
      case kOutI8:
        return SmallByKs<kOutI8>(q, small_grid, small_lds, stream);
      case kOutAcc32:
        return SmallByKs<kOutAcc32>(q, small_grid, small_lds, stream);
      default:
        return hipErrorInvalidValue;
    }
  }
  q.qpi = p.hw / 4;
  q.kgs = (4 * q.qpi + 15) / 16 * 16;  // a channel group's cells start on a 256-byte boundary: conflict-free operand reads
  q.row_groups = p.M / 128;
  const int64_t items = (int64_t)p.batch * q.row_groups;
  if (items > (1 << 28)) return hipErrorInvalidValue;
  q.items = (int)items;
  q.per_xcd = (q.items + 7) / 8;
  q.dma_full = (16 * p.hw) / 1024;
  q.dma_rem_lanes = ((16 * p.hw) % 1024) / 16;
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

}  // namespace pl
