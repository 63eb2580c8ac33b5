// fp32 walk with the whole tile and the index lists in LDS.
//
// The other fp32 walks read index lists and weights through the scalar data
// cache, whose fill rate bounds them (a list set of 70 - 100 KB per tile
// streams through a 16 KB cache; the scalar path delivers about one byte per
// clock and CU).  Here a workgroup of sixteen wavefronts keeps all input
// channels of 128 positions in LDS, and every wavefront streams the lists of
// its row groups through a private 1.5 KB LDS buffer: the next piece of the
// stream is fetched into registers with ordinary vector loads (24 bytes per
// lane) while the current one is walked, and list records are read from LDS
// with the same address in every lane.  Per entry: one 8-byte LDS read of
// the activations (two positions per lane), the entry's share of three
// 16-byte record reads, one address add and four fused multiply-adds.  A row
// group's header (rows, list length, bias) travels in the stream too, so the
// walk issues no scalar memory load.
// Outputs of a row group are stored as soon as its list ends, so the stores
// spread over the whole walk.  The order of the fused multiply-adds of one
// output is the index order and the accumulator starts at the bias, as in the
// other walks (same bits).
// With pairs (TileWalkParams::pairs) a wavefront instruction walks two row groups of about the same length at
// once: lanes 0 - 31 the first, lanes 32 - 63 the second, four positions per lane, the records of the two
// groups side by side in the stream.  The activations are then read 16 bytes per lane (LDS delivers those at
// twice the rate of 8-byte reads) and every LDS instruction, address add and loop step serves two row groups;
// the shorter group of a pair is padded with entries of weight zero at the tile's zero row.
// With more channels than a tile of 128 positions holds in LDS, the tile shrinks and a wavefront instruction walks
// more row groups, always four positions per lane: four groups on tiles of 64 positions (16 lanes each, up to 543
// channels), eight on tiles of 32 (1087), sixteen on tiles of 16 (2175).  The records of a step's groups lie side
// by side in the stream, padded to the longest list among them; the streams are made for the tile's channel rows.
// Maps whose size is not a multiple of 4 (RAGGED, not with single row groups): neighbouring positions of a tile may lie in
// different images, so the tile is staged and the outputs are stored element by element (a thread stages the
// positions c, c + 32, ... of a channel row, a lane stores each of its positions through its own address); the
// walk between the two is the same.
// With fewer tiles than CUs, the row groups can be dealt into a main and a
// spare part (two sets of sixteen streams): the tile's own workgroup walks the
// main part, and the workgroups on the CUs that have no tile of their own walk
// the spare parts of several tiles, one tile after the other.  With at most a
// third as many tiles as CUs, n workgroups share a tile with equal parts.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "epilogue.h"
#include "kernarg_head.h"
#include "launch_lds.h"
#include "sparse_conv_kernels.h"

namespace pl {
namespace {

typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(4))) uint32_t* ConstWords;
typedef const __attribute__((address_space(4))) float* ConstFloats;

// what selects the tile, picks the activation and addresses the first loads arrives in registers
PL_IN_HEAD(TileWalkParams, x);
PL_IN_HEAD(TileWalkParams, stream);
PL_IN_HEAD(TileWalkParams, stream_first);
PL_IN_HEAD(TileWalkParams, K);
PL_IN_HEAD(TileWalkParams, hw);
PL_IN_HEAD(TileWalkParams, P);
PL_IN_HEAD(TileWalkParams, tiles);
PL_IN_HEAD(TileWalkParams, split);
PL_IN_HEAD(TileWalkParams, parts);
PL_IN_HEAD(TileWalkParams, pairs);
static_assert(offsetof(TileWalkParams, act) + sizeof(int) <= kHeadWords * 8, "act.type must lie in the first 56 bytes of TileWalkParams");

using epilogue::ActivateT;
using epilogue::DispatchAct;

constexpr int kWaves = kTileWalkWaves;  // wavefronts per workgroup = list streams
constexpr int kChunkBytes = kTileWalkChunkBytes;

// One tile: stage it, then walk the streams of one part (0 main, 1 spare).
template <int NR, int ACT, int G, bool RAGGED>
__device__ __forceinline__ void WalkOneTile(const TileWalkParams& p, float* tile, int tile_id, int part) {
  // G row groups per wavefront instruction, LG lanes each
  constexpr bool PAIR = G > 1;
  constexpr int LG = 64 / G;
  constexpr int TILE = G == 1 ? kTileWalkTile : 4 * LG;
  static_assert(PAIR || !RAGGED, "maps of any size are not walked with single row groups");
  constexpr int kRecBytes = NR == 2 ? 48 : 32;  // four byte offsets, then 4 * NR weights
  constexpr int kStepBytes = G * kRecBytes;  // what one step of the walk reads: one record per row group
  constexpr int kRecs = kChunkBytes / kStepBytes;
  constexpr int PPL = PAIR ? 4 : 2;  // positions per lane
  constexpr int kTP = TILE;                  // positions per workgroup
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int sidx = part * kWaves + wave;
  const uint32_t tile0 = (uint32_t)tile_id * (uint32_t)kTP;
  char* tile_bytes = reinterpret_cast<char*>(tile);
  char* lbuf = tile_bytes + (size_t)(p.K + 1) * kTP * 4 + wave * kChunkBytes;

  // the wavefront's list stream: chunks of kChunkBytes, lane i holds bytes
  // [16 i, 16 i + 16) and [1024 + 8 i, 1024 + 8 i + 8) of a chunk
  const char* sp = reinterpret_cast<const char*>(p.stream) + (size_t)((ConstWords)p.stream_first)[sidx] * kChunkBytes;
  u4 pa = *reinterpret_cast<const u4*>(sp + 16 * lane);
  u2 pb = *reinterpret_cast<const u2*>(sp + 1024 + 8 * lane);

  // staging: kTP / 4 threads per channel row (four positions each), 32 or 64 rows per pass
  if (RAGGED) {
    constexpr int kRowThreads = kTP / 4, kPassRows = 64 * kWaves / kRowThreads;
    const int c = tid & (kRowThreads - 1), r0 = tid / kRowThreads;
    // the thread's positions c + kRowThreads * e of the tile: offset of each in channel 0 of its image
    size_t eoff[4];
    bool elive[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t pos = tile0 + (uint32_t)(c + kRowThreads * e);
      elive[e] = pos < p.P;
      const uint32_t n = elive[e] ? pos / (uint32_t)p.hw : 0u;
      const uint32_t pp = elive[e] ? pos % (uint32_t)p.hw : 0u;
      eoff[e] = (size_t)n * p.K * p.hw + pp;
    }
    for (int k0 = 0; k0 < p.K; k0 += 4 * kPassRows) {
      float v[4][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = min(k0 + r0 + kPassRows * u, p.K - 1);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[u][e] = p.x[eoff[e] + (size_t)k * p.hw];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + r0 + kPassRows * u;
        if (k < p.K) {
#pragma unroll
          for (int e = 0; e < 4; ++e) tile[(size_t)k * kTP + c + kRowThreads * e] = elive[e] ? v[u][e] : 0.0f;
        }
      }
    }
    if (tid < kTP / 4) *reinterpret_cast<uint4*>(tile_bytes + ((size_t)p.K * kTP + 4 * tid) * 4) = make_uint4(0, 0, 0, 0);
  } else {
    constexpr int kRowThreads = kTP / 4, kPassRows = 64 * kWaves / kRowThreads;
    const int c4 = tid & (kRowThreads - 1), r0 = tid / kRowThreads;
    const uint32_t gpos = tile0 + 4u * (uint32_t)c4;
    const bool live = gpos < p.P;
    const uint32_t n = live ? gpos / (uint32_t)p.hw : 0u;
    const uint32_t pp = live ? gpos % (uint32_t)p.hw : 0u;
    const float* xcol = p.x + (size_t)n * p.K * p.hw + pp;
    for (int k0 = 0; k0 < p.K; k0 += 4 * kPassRows) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = min(k0 + r0 + kPassRows * u, p.K - 1);
        v[u] = *reinterpret_cast<const uint4*>(xcol + (size_t)k * p.hw);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + r0 + kPassRows * u;
        if (k < p.K) *reinterpret_cast<uint4*>(tile_bytes + ((size_t)k * kTP + 4 * c4) * 4) = live ? v[u] : make_uint4(0, 0, 0, 0);
      }
    }
    // row K is all zero: the target of list padding entries
    if (tid < kTP / 4) *reinterpret_cast<uint4*>(tile_bytes + ((size_t)p.K * kTP + 4 * tid) * 4) = make_uint4(0, 0, 0, 0);
  }
  __syncthreads();

  // the part of the wavefront a lane belongs to picks the record, its place in the part the positions
  const int half = lane / LG;
  const uint32_t lane8 = 4u * PPL * (uint32_t)(lane & (LG - 1));
  const uint32_t gpos = tile0 + (uint32_t)PPL * (uint32_t)(lane & (LG - 1));
  const bool store_on = gpos < p.P;
  const uint32_t on = store_on ? gpos / (uint32_t)p.hw : 0u, opp = store_on ? gpos % (uint32_t)p.hw : 0u;
  float* obase = p.out + (size_t)on * p.M * p.hw + opp;
  // RAGGED: every position of the lane through its own address (row 0 of its image)
  [[maybe_unused]] float* qbase[RAGGED ? PPL : 1];
  [[maybe_unused]] bool qlive[RAGGED ? PPL : 1];
  if (RAGGED) {
#pragma unroll
    for (int q = 0; q < PPL; ++q) {
      const uint32_t pos = gpos + (uint32_t)q;
      qlive[q] = pos < p.P;
      const uint32_t n = qlive[q] ? pos / (uint32_t)p.hw : 0u, pp = qlive[q] ? pos % (uint32_t)p.hw : 0u;
      qbase[q] = p.out + (size_t)n * p.M * p.hw + pp;
    }
  }

  int rec = kRecs;  // records of the current chunk already walked: the first chunk is still in registers
  int chunk = 0;
  // next record of the stream; at the end of a chunk the prefetched one becomes
  // the current one (only this wavefront reads the buffer, and its LDS
  // operations execute in order) and the one after it is requested
  auto next = [&]() -> const char* {
    if (rec == kRecs) {
      *reinterpret_cast<u4*>(lbuf + 16 * lane) = pa;
      *reinterpret_cast<u2*>(lbuf + 1024 + 8 * lane) = pb;
      ++chunk;
      const char* np = sp + (size_t)chunk * kChunkBytes;  // the stream ends with one spare chunk
      pa = *reinterpret_cast<const u4*>(np + 16 * lane);
      pb = *reinterpret_cast<const u2*>(np + 1024 + 8 * lane);
      rec = 0;
    }
    return lbuf + (rec++) * kStepBytes + half * kRecBytes;
  };
  const int n_groups = (int)((ConstWords)p.stream_groups)[sidx];
  for (int j = 0; j < n_groups; ++j) {
    // header record of the row group: first row | rows << 24, entries, bias bits of its rows (pairs: one per half,
    // the same number of entries in both)
    const u4 hdr = *reinterpret_cast<const u4*>(next());
    const int row0 = PAIR ? (int)(hdr.x & 0xffffffu) : __builtin_amdgcn_readfirstlane((int)(hdr.x & 0xffffffu));
    const int nrows = PAIR ? (int)(hdr.x >> 24) : __builtin_amdgcn_readfirstlane((int)(hdr.x >> 24));
    const uint32_t entries = (uint32_t)__builtin_amdgcn_readfirstlane((int)hdr.y);
    float acc[NR][PPL];
#pragma unroll
    for (int q = 0; q < PPL; ++q) {
      acc[0][q] = __uint_as_float(hdr.z);
      if (NR == 2) acc[NR - 1][q] = __uint_as_float(hdr.w);
    }
    typedef float vx __attribute__((ext_vector_type(PPL)));
    auto entry = [&](uint32_t off, float w0, float w1) {
      const vx x = *reinterpret_cast<const vx*>(tile_bytes + (off + lane8));
#pragma unroll
      for (int q = 0; q < PPL; ++q) {
        acc[0][q] = __builtin_fmaf(x[q], w0, acc[0][q]);
        if (NR == 2) acc[NR - 1][q] = __builtin_fmaf(x[q], w1, acc[NR - 1][q]);
      }
    };
    auto weights = [&](const char* r, float (&w)[4 * NR]) {
      const u4 wa = *reinterpret_cast<const u4*>(r + 16);
      w[0] = __uint_as_float(wa.x), w[1] = __uint_as_float(wa.y), w[2] = __uint_as_float(wa.z), w[3] = __uint_as_float(wa.w);
      if (NR == 2) {
        const u4 wb = *reinterpret_cast<const u4*>(r + (NR == 2 ? 32 : 16));
        w[4 * NR - 4] = __uint_as_float(wb.x), w[4 * NR - 3] = __uint_as_float(wb.y), w[4 * NR - 2] = __uint_as_float(wb.z), w[4 * NR - 1] = __uint_as_float(wb.w);
      }
    };
    const uint32_t batches = entries >> 2, rem = entries & 3u;
    for (uint32_t b = 0; b < batches; ++b) {
      const char* r = next();
      const u4 off = *reinterpret_cast<const u4*>(r);
      float w[4 * NR];
      weights(r, w);
      vx x[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = *reinterpret_cast<const vx*>(tile_bytes + (off[e] + lane8));
#pragma unroll
      for (int e = 0; e < 4; ++e) {
#pragma unroll
        for (int q = 0; q < PPL; ++q) {
          acc[0][q] = __builtin_fmaf(x[e][q], w[e * NR], acc[0][q]);
          if (NR == 2) acc[NR - 1][q] = __builtin_fmaf(x[e][q], w[e * NR + NR - 1], acc[NR - 1][q]);
        }
      }
    }
    if (rem != 0) {  // the last, partly filled batch: only its real entries
      const char* r = next();
      const u4 off = *reinterpret_cast<const u4*>(r);
      float w[4 * NR];
      weights(r, w);
      entry(off[0], w[0], w[NR - 1]);
      if (rem > 1) entry(off[1], w[NR], w[NR + NR - 1]);
      if (rem > 2) entry(off[2], w[2 * NR], w[2 * NR + NR - 1]);
    }
    if (RAGGED) {
#pragma unroll
      for (int rr = 0; rr < NR; ++rr) {
        if (rr < nrows) {
          const size_t at = (size_t)(row0 + rr) * p.hw;
#pragma unroll
          for (int q = 0; q < PPL; ++q)
            if (qlive[q]) qbase[q][at] = ActivateT<ACT>(acc[rr][q], p.act);
        }
      }
    } else if (store_on) {
#pragma unroll
      for (int rr = 0; rr < NR; ++rr) {
        if (rr < nrows) {
          vx o;
#pragma unroll
          for (int q = 0; q < PPL; ++q) o[q] = ActivateT<ACT>(acc[rr][q], p.act);
          __builtin_nontemporal_store(o, reinterpret_cast<vx*>(obase + (size_t)(row0 + rr) * p.hw));
        }
      }
    }
  }
}

// Workgroup id -> tiles: each XCD (linear id mod 8) owns a contiguous range of
// tiles.  Its first workgroups take one tile each (main part); with a spare
// part, the workgroups behind them share the range's tiles among themselves.
template <int NR, int ACT, int G, bool RAGGED>
__device__ __forceinline__ void TileWalkBody(const TileWalkParams& p, float* tile) {
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int first = (xcd * p.tiles) >> 3, last = ((xcd + 1) * p.tiles) >> 3;
  const int count = last - first;
  if (p.split == 2) {
    // equal parts: part = slot / count of tile slot % count
    const int part = count > 0 ? slot / count : p.parts;
    if (part < p.parts) WalkOneTile<NR, ACT, G, RAGGED>(p, tile, first + (slot - part * count), part);
    return;
  }
  if (slot < count) {
    WalkOneTile<NR, ACT, G, RAGGED>(p, tile, first + slot, 0);
    return;
  }
  if (p.split == 0) return;
  const int n_spare = (int)(gridDim.x >> 3) - count;
  for (int t = first + (slot - count); t < last; t += n_spare) {
    WalkOneTile<NR, ACT, G, RAGGED>(p, tile, t, 1);
    __syncthreads();  // every wavefront has left the tile before the next one is staged
  }
}

template <int NR>
__global__ void __launch_bounds__(64 * kTileWalkWaves) TileWalkKernel(PL_HEAD_PARAMS, const TileWalkParams block) {
  const TileWalkParams p = WithHead(block, PL_HEAD_ARGS);
  extern __shared__ float tile_lds[];
  DispatchAct(p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    switch (p.pairs) {
      case 0:
        TileWalkBody<NR, ACT, 1, false>(p, tile_lds);
        break;
      case 1:
        TileWalkBody<NR, ACT, 2, false>(p, tile_lds);
        break;
      case 2:
        TileWalkBody<NR, ACT, 4, false>(p, tile_lds);
        break;
      case 3:
        TileWalkBody<NR, ACT, 8, false>(p, tile_lds);
        break;
      case 4:
        TileWalkBody<NR, ACT, 16, false>(p, tile_lds);
        break;
      case 1 | kTileWalkRagged:
        TileWalkBody<NR, ACT, 2, true>(p, tile_lds);
        break;
      case 2 | kTileWalkRagged:
        TileWalkBody<NR, ACT, 4, true>(p, tile_lds);
        break;
      case 3 | kTileWalkRagged:
        TileWalkBody<NR, ACT, 8, true>(p, tile_lds);
        break;
      default:  // 4 | kTileWalkRagged
        TileWalkBody<NR, ACT, 16, true>(p, tile_lds);
        break;
    }
  });
}

}  // namespace

size_t TileWalkLdsBytes(int K, int row_bytes) { return (size_t)(K + 1) * (size_t)row_bytes + (size_t)kWaves * kChunkBytes; }

hipError_t LaunchTileWalk(int nrows, const TileWalkParams& p, hipStream_t stream) {
  if (p.P == 0 || p.n_groups == 0) return hipSuccess;
  const int form = p.pairs & (kTileWalkRagged - 1);
  const bool ragged = (p.pairs & kTileWalkRagged) != 0;
  if (form > 4 || (ragged && form == 0) || (!ragged && p.hw % 4 != 0)) return hipErrorInvalidValue;
  const int tile = TileWalkTileOf(form);
  const size_t lds = TileWalkLdsBytes(p.K, tile * 4);
  if (lds > (size_t)kMaxLdsBytes) return hipErrorInvalidValue;
  TileWalkParams q = p;
  q.tiles = (int)((p.P + (uint32_t)tile - 1) / (uint32_t)tile);
  uint32_t slots = ((uint32_t)q.tiles + 7) / 8;  // workgroups per XCD
  if (q.split == 2) {
    if (q.parts < 2 || (int64_t)q.parts * slots > q.split_slots) return hipErrorInvalidValue;
    slots *= (uint32_t)q.parts;
  } else if (q.split != 0) {
    if (q.split_slots < (int)slots + 1) return hipErrorInvalidValue;  // every XCD needs a spare workgroup
    slots = (uint32_t)q.split_slots;
  }
  dim3 grid(8u * slots), block(64 * kWaves);
  if (nrows == 2) return LaunchWithHead(TileWalkKernel<2>, grid, block, lds, stream, q);
  return LaunchWithHead(TileWalkKernel<1>, grid, block, lds, stream, q);
}

}  // namespace pl
