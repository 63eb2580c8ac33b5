// Row walk in half precision: activations, weights, bias, accumulators and
// the activation function are all IEEE binary16, one rounding per
// instruction (v_pk_fma_f16 for the multiply-accumulate), in index order.
//
// A workgroup stages a tile of TP positions x all channels in LDS
// ([channel][position] halves plus one all-zero row for the padding entries
// of the index lists); a wavefront owns one output row (or row pair) at a
// time, a lane two neighbouring positions.  Index lists and weights are read
// through the constant address space (scalar loads).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernarg_head.h"
#include "launch_lds.h"
#include "sparse_conv_kernels.h"

namespace pl {
namespace {

typedef _Float16 h1;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(4))) uint32_t* ConstWords;
typedef const __attribute__((address_space(4))) uint16_t* ConstHalves;

__device__ __forceinline__ h1 HalfBits(uint16_t b) { return __builtin_bit_cast(h1, b); }
__device__ __forceinline__ uint16_t BitsOf(h1 v) { return __builtin_bit_cast(uint16_t, v); }
__device__ __forceinline__ h2 Both(h1 v) { return h2{v, v}; }

__device__ __forceinline__ int XcdTile(int tiles, int per_tile) {
  const int xcd = blockIdx.x & 7, wg_slot = blockIdx.x >> 3;
  const int first = (xcd * tiles) >> 3, last = ((xcd + 1) * tiles) >> 3;
  const int t = first + wg_slot / per_tile;
  return t < last ? t : -1;
}

// Activation on two values, every step its own half-precision instruction:
// relu max(v,0); relu6 min(max(v,0),six); leaky v >= 0 ? v : v*alpha;
// hard_swish (v * (1/scale)) * min(max(v + offset, 0), threshold).
template <int ACT>
__device__ __forceinline__ h2 ActivateH(h2 v, const DevActH& a) {
  const h2 zero = {(h1)0, (h1)0};
  if (ACT == 1) return __builtin_elementwise_max(v, zero);
  if (ACT == 2) return __builtin_elementwise_min(__builtin_elementwise_max(v, zero), Both(HalfBits(a.alpha)));
  if (ACT == 4) {
    const h2 m = v * Both(HalfBits(a.alpha));
    return h2{v.x >= (h1)0 ? v.x : m.x, v.y >= (h1)0 ? v.y : m.y};
  }
  if (ACT == 10) {
    h2 t = v + Both(HalfBits(a.hs_offset));
    const h2 u = v * Both(HalfBits(a.hs_inv_scale));
    t = __builtin_elementwise_min(__builtin_elementwise_max(t, zero), Both(HalfBits(a.hs_threshold)));
    return u * t;
  }
  return v;
}

template <int NR, int TP, int ACT>
__device__ __forceinline__ void HalfWalkBody(const HalfWalkParams& p, uint32_t* tile32) {
  uint16_t* tile = reinterpret_cast<uint16_t*>(tile32);
  const int tile_id = XcdTile(p.tiles, p.slices);
  if (tile_id < 0) return;
  const int slice = (blockIdx.x >> 3) % p.slices;
  const uint32_t tile0 = (uint32_t)tile_id * (uint32_t)TP;
  const int tid = threadIdx.x, nthreads = blockDim.x;

  // ---- staging: [channel][TP] halves; row K is zero
  if (p.pair) {
    // positions two at a time (hw even, x 4-byte aligned: a pair never
    // leaves its image)
    constexpr int TP2 = TP / 2;
    const int j2 = tid % TP2;
    const uint32_t g = tile0 + 2u * j2;
    const bool live = g < p.P;
    const uint32_t n = live ? g / (uint32_t)p.hw : 0u, pp = live ? g % (uint32_t)p.hw : 0u;
    const uint16_t* col = p.x + (size_t)n * p.K * p.hw + pp;
    for (int k = tid / TP2; k <= p.K; k += nthreads / TP2) {
      uint32_t v = 0;
      if (live && k < p.K) v = *reinterpret_cast<const uint32_t*>(col + (size_t)k * p.hw);
      tile32[(size_t)k * TP2 + j2] = v;
    }
  } else {
    const int j = tid % TP;
    const uint32_t g = tile0 + j;
    const bool live = g < p.P;
    const uint32_t n = live ? g / (uint32_t)p.hw : 0u, pp = live ? g % (uint32_t)p.hw : 0u;
    const uint16_t* col = p.x + (size_t)n * p.K * p.hw + pp;
    for (int k = tid / TP; k <= p.K; k += nthreads / TP) tile[(size_t)k * TP + j] = (live && k < p.K) ? col[(size_t)k * p.hw] : (uint16_t)0;
  }
  __syncthreads();

  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nwaves = nthreads >> 6;
  const bool lane_on = 2 * lane < TP;
  const uint32_t* xlane = tile32 + (lane_on ? lane : 0);  // the lane's two positions of channel 0
  const ConstWords group_words = (ConstWords)p.groups;
  const ConstWords kidx = (ConstWords)p.kidx;
  const ConstWords wts = (ConstWords)p.wts;
  const ConstHalves bias = (ConstHalves)p.bias;
  const int g_begin = slice * p.groups_per_slice;
  const int g_end = min(p.n_groups, g_begin + p.groups_per_slice);

  for (int g = g_begin + wave; g < g_end; g += nwaves) {
    const ConstWords gw = group_words + (size_t)g * 4;
    const int row0 = (int)gw[0], nrows = (int)gw[1];
    const uint32_t first = gw[2], count = gw[3];
    h2 a0 = {(h1)0, (h1)0}, a1 = {(h1)0, (h1)0};
    if (bias) {
      a0 = Both(HalfBits(bias[row0]));
      if (NR == 2 && nrows == 2) a1 = Both(HalfBits(bias[row0 + 1]));
    }
    const ConstWords kp = kidx + first;
    const ConstWords wp = wts + first;
    // list lengths are multiples of kWalkBatch
    for (uint32_t e = 0; e < count; e += kWalkBatch) {
#pragma unroll
      for (int i = 0; i < kWalkBatch; ++i) {
        const uint32_t k = kp[e + i], w = wp[e + i];
        const h2 xv = __builtin_bit_cast(h2, xlane[(size_t)k * (TP / 2)]);
        a0 = __builtin_elementwise_fma(xv, Both(HalfBits((uint16_t)(w & 0xffffu))), a0);
        if (NR == 2) a1 = __builtin_elementwise_fma(xv, Both(HalfBits((uint16_t)(w >> 16))), a1);
      }
    }
    if (!lane_on) continue;
    const uint32_t gpos = tile0 + 2u * (uint32_t)lane;
    if (gpos >= p.P) continue;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (r < nrows) {
        const h2 v = ActivateH<ACT>(r == 0 ? a0 : a1, p.act);
        const int row = row0 + r;
        if (p.pair) {
          const uint32_t n = gpos / (uint32_t)p.hw, pp = gpos % (uint32_t)p.hw;
          __builtin_nontemporal_store(__builtin_bit_cast(uint32_t, v), reinterpret_cast<uint32_t*>(p.out + ((size_t)n * p.M + row) * p.hw + pp));
        } else {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const uint32_t gj = gpos + j;
            if (gj < p.P) {
              const uint32_t n = gj / (uint32_t)p.hw, pp = gj % (uint32_t)p.hw;
              p.out[((size_t)n * p.M + row) * p.hw + pp] = BitsOf(j == 0 ? v.x : v.y);
            }
          }
        }
      }
    }
  }
}

template <int NR, int TP>
__global__ void __launch_bounds__(1024) HalfWalkKernel(const HalfWalkParams p) {
  extern __shared__ uint32_t tile32[];
  switch (p.act.type) {
    case 1:
      HalfWalkBody<NR, TP, 1>(p, tile32);
      break;
    case 2:
      HalfWalkBody<NR, TP, 2>(p, tile32);
      break;
    case 4:
      HalfWalkBody<NR, TP, 4>(p, tile32);
      break;
    case 10:
      HalfWalkBody<NR, TP, 10>(p, tile32);
      break;
    default:
      HalfWalkBody<NR, TP, 0>(p, tile32);
      break;
  }
}

// ------------------------------------------------- walk over channel chunks
// The half-precision counterpart of the fp32 walk over channel chunks: a
// workgroup (8 wavefronts) takes 256 positions and stages the channels 64 at
// a time; a wavefront keeps the accumulators of its G row groups in registers
// across the chunks and walks, per chunk, the entries whose channel lies in
// it; a lane works on four consecutive positions (one 8-byte LDS read and two
// packed multiply-adds per entry and row).  One list fetch serves 256
// positions whatever the channel count.  The multiply-adds of one output keep
// the index order.
constexpr int kCChunk = kChunkWalkChunk;
constexpr int kCWaves = kChunkWalkWaves;

// PPL: positions per lane (4 or 8); the tile has 64 * PPL positions.
template <int PPL>
struct LanePiece;
template <>
struct LanePiece<4> {
  typedef uint2 type;
};
template <>
struct LanePiece<8> {
  typedef uint4 type;
};

template <int NR, int G, int PPL, int ACT>
__device__ __forceinline__ void HalfChunkWalkBody(const HalfChunkWalkParams& p, uint32_t* tile32) {
  constexpr int kTile = 64 * PPL;     // positions per workgroup
  constexpr int kRowWords = kTile / 2;  // dwords per LDS row
  constexpr int kLaneWords = PPL / 2;   // dwords (pairs of positions) per lane
  typedef typename LanePiece<PPL>::type Piece;
  const int tile_id = XcdTile(p.tiles, p.slices);
  if (tile_id < 0) return;
  const int slice = (blockIdx.x >> 3) % p.slices;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t tile0 = (uint32_t)tile_id * (uint32_t)kTile;
  const ConstWords group_words = (ConstWords)p.groups;
  const ConstHalves biasp = (ConstHalves)p.bias;
  const ConstWords descp = (ConstWords)p.desc;
  const ConstWords idxp = (ConstWords)p.idx;
  const ConstWords wtsp = (ConstWords)p.wts;

  const int g_first = (slice * kCWaves + wave) * G;
  h2 acc[G][NR][kLaneWords];
#pragma unroll
  for (int gi = 0; gi < G; ++gi) {
    const int g = g_first + gi;
    h1 b0 = (h1)0, b1 = (h1)0;
    if (g < p.n_groups && biasp) {
      const int row0 = (int)group_words[(size_t)g * 4], nrows = (int)group_words[(size_t)g * 4 + 1];
      b0 = HalfBits(biasp[row0]);
      if (NR == 2 && nrows == 2) b1 = HalfBits(biasp[row0 + 1]);
    }
#pragma unroll
    for (int j = 0; j < kLaneWords; ++j) {
      acc[gi][0][j] = Both(b0);
      if (NR == 2) acc[gi][NR - 1][j] = Both(b1);
    }
  }

  // staging: thread = (PPL positions, channel row of a pass of 8 rows)
  const int jl = tid & 63, r0 = tid >> 6;
  const uint32_t gpos = tile0 + (uint32_t)PPL * (uint32_t)jl;
  const bool live = gpos < p.P;
  const uint32_t n = live ? gpos / (uint32_t)p.hw : 0u;
  const uint32_t pp = live ? gpos % (uint32_t)p.hw : 0u;
  const uint16_t* xcol = p.x + (size_t)n * p.K * p.hw + pp;
  const uint32_t* xlane = tile32 + kLaneWords * lane;  // the lane's positions of LDS row 0
  Piece zero;
  __builtin_memset(&zero, 0, sizeof(zero));

  for (int chunk = 0; chunk < p.n_chunks; ++chunk) {
    if (chunk > 0) __syncthreads();  // the previous chunk is read until every wavefront has walked it
    {
      const int c0 = chunk * kCChunk;
      Piece v[kCChunk / kCWaves];
#pragma unroll
      for (int u = 0; u < kCChunk / kCWaves; ++u) {
        const int ch = min(c0 + r0 + kCWaves * u, p.K - 1);
        v[u] = *reinterpret_cast<const Piece*>(xcol + (size_t)ch * p.hw);
      }
#pragma unroll
      for (int u = 0; u < kCChunk / kCWaves; ++u) {
        const int kl = r0 + kCWaves * u;
        const bool on = live && c0 + kl < p.K;
        *reinterpret_cast<Piece*>(tile32 + (size_t)kl * kRowWords + kLaneWords * jl) = on ? v[u] : zero;
      }
      // row kCChunk is all zero: the target of list padding entries
      if (chunk == 0 && tid < 64) *reinterpret_cast<Piece*>(tile32 + (size_t)kCChunk * kRowWords + kLaneWords * tid) = zero;
    }
    __syncthreads();

    const ConstWords dw = descp + ((size_t)((slice * p.n_chunks + chunk) * kCWaves + wave) * G) * 2;
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
      const uint32_t first = dw[2 * gi], batches = dw[2 * gi + 1];
      const ConstWords ip = idxp + first;
      const ConstWords wp = wtsp + (size_t)first * 4;
      for (uint32_t b = 0; b < batches; ++b) {
        const uint32_t packed = ip[b];
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = wp[(size_t)b * 4 + i];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t kl = (packed >> (8 * e)) & 0xffu;
          const Piece xv = *reinterpret_cast<const Piece*>(xlane + (size_t)kl * kRowWords);
          uint32_t xw[kLaneWords];
          __builtin_memcpy(xw, &xv, sizeof(xv));
          const h2 w0 = Both(HalfBits((uint16_t)(w[e] & 0xffffu)));
          const h2 w1 = Both(HalfBits((uint16_t)(w[e] >> 16)));
#pragma unroll
          for (int j = 0; j < kLaneWords; ++j) {
            const h2 x2 = __builtin_bit_cast(h2, xw[j]);
            acc[gi][0][j] = __builtin_elementwise_fma(x2, w0, acc[gi][0][j]);
            if (NR == 2) acc[gi][NR - 1][j] = __builtin_elementwise_fma(x2, w1, acc[gi][NR - 1][j]);
          }
        }
      }
    }
  }

  const uint32_t opos = tile0 + (uint32_t)PPL * (uint32_t)lane;
  if (opos >= p.P) return;
  const uint32_t on = opos / (uint32_t)p.hw, opp = opos % (uint32_t)p.hw;
#pragma unroll
  for (int gi = 0; gi < G; ++gi) {
    const int g = g_first + gi;
    if (g >= p.n_groups) break;
    const int row0 = (int)group_words[(size_t)g * 4], nrows = (int)group_words[(size_t)g * 4 + 1];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (r < nrows) {
        typedef uint32_t vNu __attribute__((ext_vector_type(kLaneWords)));
        vNu o;
#pragma unroll
        for (int j = 0; j < kLaneWords; ++j) o[j] = __builtin_bit_cast(uint32_t, ActivateH<ACT>(acc[gi][r][j], p.act));
        uint16_t* dst = p.out + ((size_t)on * p.M + row0 + r) * p.hw + opp;
        __builtin_nontemporal_store(o, reinterpret_cast<vNu*>(dst));
      }
    }
  }
}

template <int NR, int G, int PPL>
__global__ void __launch_bounds__(64 * kChunkWalkWaves, 2) HalfChunkWalkKernel(const HalfChunkWalkParams p) {
  extern __shared__ uint32_t tile32[];
  switch (p.act.type) {
    case 1:
      HalfChunkWalkBody<NR, G, PPL, 1>(p, tile32);
      break;
    case 2:
      HalfChunkWalkBody<NR, G, PPL, 2>(p, tile32);
      break;
    case 4:
      HalfChunkWalkBody<NR, G, PPL, 4>(p, tile32);
      break;
    case 10:
      HalfChunkWalkBody<NR, G, PPL, 10>(p, tile32);
      break;
    default:
      HalfChunkWalkBody<NR, G, PPL, 0>(p, tile32);
      break;
  }
}

// Walk with the whole tile and the index lists in LDS (the structure of the fp32 tile walk with pairs of row
// groups): a workgroup of sixteen wavefronts keeps all channels of 256 positions in LDS, 512 bytes per channel
// row, and every wavefront streams the double records of its pairs of row groups through a private LDS buffer.
// Lanes 0 - 31 walk the first row group of a pair, lanes 32 - 63 the second, eight positions per lane: per
// entry one 16-byte LDS read and four v_pk_fma_f16 per row.  (PPL = 4: tiles of 128 positions, four per lane,
// 8-byte reads and two v_pk_fma_f16 - for channel counts whose wide tile does not fit LDS and for maps whose size
// is a multiple of 4 only.)  Weights and biases arrive in the stream as
// binary16 values doubled into a dword, so they need no splat.  The accumulator of an output starts at its
// bias and takes its entries in index order, one rounding per entry, as in the other half-precision walks
// (same bits).
PL_IN_HEAD(HalfTileWalkParams, x);
PL_IN_HEAD(HalfTileWalkParams, stream);
PL_IN_HEAD(HalfTileWalkParams, stream_first);
PL_IN_HEAD(HalfTileWalkParams, K);
PL_IN_HEAD(HalfTileWalkParams, hw);
PL_IN_HEAD(HalfTileWalkParams, P);
PL_IN_HEAD(HalfTileWalkParams, tiles);
PL_IN_HEAD(HalfTileWalkParams, split);
PL_IN_HEAD(HalfTileWalkParams, parts);
static_assert(offsetof(HalfTileWalkParams, act) + sizeof(int) <= kHeadWords * 8, "act.type must lie in the first 56 bytes of HalfTileWalkParams");

typedef uint32_t u2w __attribute__((ext_vector_type(2)));
typedef uint32_t u4w __attribute__((ext_vector_type(4)));
constexpr int kTwWaves = kTileWalkWaves;
constexpr int kTwChunkBytes = kTileWalkChunkBytes;
static_assert(kHalfTileWalkTile * 2 == kTileWalkTile * 4, "the wide tile's list streams hold the byte offsets of the fp32 walk's channel rows");

// what a lane holds of a channel row: PPL positions
template <int PPL>
struct TwPiece;
template <>
struct TwPiece<8> {
  typedef u4w type;
};
template <>
struct TwPiece<4> {
  typedef u2w type;
};

// One tile: stage it, then walk the streams of one part (0 main, 1 spare).
// RAGGED: the map size is not a multiple of the lane's piece (or the tensors are not aligned to it), so the tile is
// staged and the outputs are stored one binary16 value at a time, each through its own address.
// G row groups per wavefront instruction (LG = 64 / G lanes each) on tiles of LG * PPL positions.
template <int NR, int G, int PPL, int ACT, bool RAGGED>
__device__ __forceinline__ void HalfWalkOneTile(const HalfTileWalkParams& p, char* tile_bytes, int tile_id, int part) {
  typedef typename TwPiece<PPL>::type Piece;
  constexpr int LG = 64 / G, kPassRows = 64 * kTwWaves / LG;
  constexpr int kTwTile = LG * PPL, kTwRowBytes = kTwTile * 2, kPieceBytes = 2 * PPL, NW = PPL / 2;
  constexpr int kRecBytes = NR == 2 ? 48 : 32;  // four byte offsets, then 4 * NR doubled weights
  constexpr int kStepBytes = G * kRecBytes;     // one record per row group of the step
  constexpr int kRecs = kTwChunkBytes / kStepBytes;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int sidx = part * kTwWaves + wave;
  const uint32_t tile0 = (uint32_t)tile_id * (uint32_t)kTwTile;
  char* lbuf = tile_bytes + (size_t)(p.K + 1) * kTwRowBytes + wave * kTwChunkBytes;

  // the wavefront's list stream: chunks of kTwChunkBytes, lane i holds bytes [16 i, 16 i + 16) and
  // [1024 + 8 i, 1024 + 8 i + 8) of a chunk
  const char* sp = reinterpret_cast<const char*>(p.stream) + (size_t)((ConstWords)p.stream_first)[sidx] * kTwChunkBytes;
  u4w pa = *reinterpret_cast<const u4w*>(sp + 16 * lane);
  u2w pb = *reinterpret_cast<const u2w*>(sp + 1024 + 8 * lane);

  // staging: LG threads per channel row (PPL positions each), kPassRows rows per pass
  if (RAGGED) {
    const int c = tid & (LG - 1), r0 = tid / LG;
    // the thread's positions c + LG e of the tile: offset of each in channel 0 of its image
    size_t eoff[PPL];
    bool elive[PPL];
#pragma unroll
    for (int e = 0; e < PPL; ++e) {
      const uint32_t pos = tile0 + (uint32_t)(c + LG * e);
      elive[e] = pos < p.P;
      const uint32_t n = elive[e] ? pos / (uint32_t)p.hw : 0u;
      const uint32_t pp = elive[e] ? pos % (uint32_t)p.hw : 0u;
      eoff[e] = (size_t)n * p.K * p.hw + pp;
    }
    uint16_t* tile16 = reinterpret_cast<uint16_t*>(tile_bytes);
    for (int k0 = 0; k0 < p.K; k0 += 4 * kPassRows) {
      uint16_t v[4][PPL];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = min(k0 + r0 + kPassRows * u, p.K - 1);
#pragma unroll
        for (int e = 0; e < PPL; ++e) v[u][e] = p.x[eoff[e] + (size_t)k * p.hw];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + r0 + kPassRows * u;
        if (k < p.K) {
#pragma unroll
          for (int e = 0; e < PPL; ++e) tile16[(size_t)k * kTwTile + c + LG * e] = elive[e] ? v[u][e] : (uint16_t)0;
        }
      }
    }
    Piece zero;
    __builtin_memset(&zero, 0, sizeof(zero));
    if (tid < LG) *reinterpret_cast<Piece*>(tile_bytes + (size_t)p.K * kTwRowBytes + kPieceBytes * tid) = zero;
  } else {
    const int c8 = tid & (LG - 1), r0 = tid / LG;
    const uint32_t gpos = tile0 + (uint32_t)PPL * (uint32_t)c8;
    const bool live = gpos < p.P;
    const uint32_t n = live ? gpos / (uint32_t)p.hw : 0u;
    const uint32_t pp = live ? gpos % (uint32_t)p.hw : 0u;
    const uint16_t* xcol = p.x + (size_t)n * p.K * p.hw + pp;
    Piece zero;
    __builtin_memset(&zero, 0, sizeof(zero));
    for (int k0 = 0; k0 < p.K; k0 += 4 * kPassRows) {
      Piece v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = min(k0 + r0 + kPassRows * u, p.K - 1);
        v[u] = *reinterpret_cast<const Piece*>(xcol + (size_t)k * p.hw);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + r0 + kPassRows * u;
        if (k < p.K) *reinterpret_cast<Piece*>(tile_bytes + (size_t)k * kTwRowBytes + kPieceBytes * c8) = live ? v[u] : zero;
      }
    }
    // row K is all zero: the target of list padding entries
    if (tid < LG) *reinterpret_cast<Piece*>(tile_bytes + (size_t)p.K * kTwRowBytes + kPieceBytes * tid) = zero;
  }
  __syncthreads();

  const int half = lane / LG;
  const uint32_t lane16 = (uint32_t)kPieceBytes * (uint32_t)(lane & (LG - 1));
  const uint32_t gpos = tile0 + (uint32_t)PPL * (uint32_t)(lane & (LG - 1));
  const bool store_on = gpos < p.P;
  const uint32_t on = store_on ? gpos / (uint32_t)p.hw : 0u, opp = store_on ? gpos % (uint32_t)p.hw : 0u;
  uint16_t* obase = p.out + (size_t)on * p.M * p.hw + opp;
  // RAGGED: every position of the lane through its own address (row 0 of its image)
  [[maybe_unused]] uint16_t* qbase[RAGGED ? PPL : 1];
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
  // next double record of the stream; at the end of a chunk the prefetched one becomes the current one (only
  // this wavefront reads the buffer, and its LDS operations execute in order) and the one after it is requested
  auto next = [&]() -> const char* {
    if (rec == kRecs) {
      *reinterpret_cast<u4w*>(lbuf + 16 * lane) = pa;
      *reinterpret_cast<u2w*>(lbuf + 1024 + 8 * lane) = pb;
      ++chunk;
      const char* np = sp + (size_t)chunk * kTwChunkBytes;  // the stream ends with one spare chunk
      pa = *reinterpret_cast<const u4w*>(np + 16 * lane);
      pb = *reinterpret_cast<const u2w*>(np + 1024 + 8 * lane);
      rec = 0;
    }
    return lbuf + (rec++) * kStepBytes + half * kRecBytes;
  };
  const int n_groups = (int)((ConstWords)p.stream_groups)[sidx];
  for (int j = 0; j < n_groups; ++j) {
    // header record of a row group: first row | rows << 24, entries (the same in both halves), doubled bias
    // of its rows
    const u4w hdr = *reinterpret_cast<const u4w*>(next());
    const int row0 = (int)(hdr.x & 0xffffffu);
    const int nrows = (int)(hdr.x >> 24);
    const uint32_t entries = (uint32_t)__builtin_amdgcn_readfirstlane((int)hdr.y);
    // (bit casts take scalars: applied to an element of a vector they read its first element)
    const uint32_t bias0 = hdr.z, bias1 = hdr.w;
    h2 acc[NR][NW];
#pragma unroll
    for (int q = 0; q < NW; ++q) {
      acc[0][q] = __builtin_bit_cast(h2, bias0);
      if (NR == 2) acc[NR - 1][q] = __builtin_bit_cast(h2, bias1);
    }
    auto entry = [&](const Piece& x, uint32_t w0, uint32_t w1) {
#pragma unroll
      for (int q = 0; q < NW; ++q) {
        const uint32_t xq = x[q];
        const h2 x2 = __builtin_bit_cast(h2, xq);
        acc[0][q] = __builtin_elementwise_fma(x2, __builtin_bit_cast(h2, w0), acc[0][q]);
        if (NR == 2) acc[NR - 1][q] = __builtin_elementwise_fma(x2, __builtin_bit_cast(h2, w1), acc[NR - 1][q]);
      }
    };
    auto weights = [&](const char* r, uint32_t (&w)[4 * NR]) {
      const u4w wa = *reinterpret_cast<const u4w*>(r + 16);
      w[0] = wa.x, w[1] = wa.y, w[2] = wa.z, w[3] = wa.w;
      if (NR == 2) {
        const u4w wb = *reinterpret_cast<const u4w*>(r + (NR == 2 ? 32 : 16));
        w[4 * NR - 4] = wb.x, w[4 * NR - 3] = wb.y, w[4 * NR - 2] = wb.z, w[4 * NR - 1] = wb.w;
      }
    };
    const uint32_t batches = entries >> 2, rem = entries & 3u;
    for (uint32_t b = 0; b < batches; ++b) {
      const char* r = next();
      const u4w off = *reinterpret_cast<const u4w*>(r);
      uint32_t w[4 * NR];
      weights(r, w);
      Piece x[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = *reinterpret_cast<const Piece*>(tile_bytes + (off[e] + lane16));
#pragma unroll
      for (int e = 0; e < 4; ++e) entry(x[e], w[e * NR], w[e * NR + NR - 1]);
    }
    if (rem != 0) {  // the last, partly filled batch: only its real entries
      const char* r = next();
      const u4w off = *reinterpret_cast<const u4w*>(r);
      uint32_t w[4 * NR];
      weights(r, w);
      entry(*reinterpret_cast<const Piece*>(tile_bytes + (off[0] + lane16)), w[0], w[NR - 1]);
      if (rem > 1) entry(*reinterpret_cast<const Piece*>(tile_bytes + (off[1] + lane16)), w[NR], w[NR + NR - 1]);
      if (rem > 2) entry(*reinterpret_cast<const Piece*>(tile_bytes + (off[2] + lane16)), w[2 * NR], w[2 * NR + NR - 1]);
    }
    if (RAGGED) {
#pragma unroll
      for (int rr = 0; rr < NR; ++rr) {
        if (rr < nrows) {
          const size_t at = (size_t)(row0 + rr) * p.hw;
#pragma unroll
          for (int q = 0; q < NW; ++q) {
            const h2 o = ActivateH<ACT>(acc[rr][q], p.act);
            if (qlive[2 * q]) qbase[2 * q][at] = BitsOf(o.x);
            if (qlive[2 * q + 1]) qbase[2 * q + 1][at] = BitsOf(o.y);
          }
        }
      }
    } else if (store_on) {
#pragma unroll
      for (int rr = 0; rr < NR; ++rr) {
        if (rr < nrows) {
          Piece o;
#pragma unroll
          for (int q = 0; q < NW; ++q) o[q] = __builtin_bit_cast(uint32_t, ActivateH<ACT>(acc[rr][q], p.act));
          __builtin_nontemporal_store(o, reinterpret_cast<Piece*>(obase + (size_t)(row0 + rr) * p.hw));
        }
      }
    }
  }
}

// Workgroup id -> tiles, as in the fp32 tile walk: each XCD (linear id mod 8) owns a contiguous range of tiles;
// its first workgroups take one tile each (main part), with a spare part the workgroups behind them share the
// range's tiles among themselves, with equal parts `parts` workgroups share every tile.
template <int NR, int G, int PPL, int ACT, bool RAGGED>
__device__ __forceinline__ void HalfTileWalkBody(const HalfTileWalkParams& p, char* tile) {
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int first = (xcd * p.tiles) >> 3, last = ((xcd + 1) * p.tiles) >> 3;
  const int count = last - first;
  if (p.split == 2) {
    const int part = count > 0 ? slot / count : p.parts;
    if (part < p.parts) HalfWalkOneTile<NR, G, PPL, ACT, RAGGED>(p, tile, first + (slot - part * count), part);
    return;
  }
  if (slot < count) {
    HalfWalkOneTile<NR, G, PPL, ACT, RAGGED>(p, tile, first + slot, 0);
    return;
  }
  if (p.split == 0) return;
  const int n_spare = (int)(gridDim.x >> 3) - count;
  for (int t = first + (slot - count); t < last; t += n_spare) {
    HalfWalkOneTile<NR, G, PPL, ACT, RAGGED>(p, tile, t, 1);
    __syncthreads();  // every wavefront has left the tile before the next one is staged
  }
}

template <int NR, int G, int PPL>
__global__ void __launch_bounds__(64 * kTileWalkWaves) HalfTileWalkKernel(PL_HEAD_PARAMS, const HalfTileWalkParams block) {
  const HalfTileWalkParams p = WithHead(block, PL_HEAD_ARGS);
  extern __shared__ uint32_t tile32[];
  char* tile = reinterpret_cast<char*>(tile32);
  switch (p.act.type) {
    case 1:
      if (p.form & kTileWalkRagged) {
        HalfTileWalkBody<NR, G, PPL, 1, true>(p, tile);
      } else {
        HalfTileWalkBody<NR, G, PPL, 1, false>(p, tile);
      }
      break;
    case 2:
      if (p.form & kTileWalkRagged) {
        HalfTileWalkBody<NR, G, PPL, 2, true>(p, tile);
      } else {
        HalfTileWalkBody<NR, G, PPL, 2, false>(p, tile);
      }
      break;
    case 4:
      if (p.form & kTileWalkRagged) {
        HalfTileWalkBody<NR, G, PPL, 4, true>(p, tile);
      } else {
        HalfTileWalkBody<NR, G, PPL, 4, false>(p, tile);
      }
      break;
    case 10:
      if (p.form & kTileWalkRagged) {
        HalfTileWalkBody<NR, G, PPL, 10, true>(p, tile);
      } else {
        HalfTileWalkBody<NR, G, PPL, 10, false>(p, tile);
      }
      break;
    default:
      if (p.form & kTileWalkRagged) {
        HalfTileWalkBody<NR, G, PPL, 0, true>(p, tile);
      } else {
        HalfTileWalkBody<NR, G, PPL, 0, false>(p, tile);
      }
      break;
  }
}

template <typename K>
hipError_t LaunchBig(K kernel, dim3 grid, dim3 block, size_t lds, hipStream_t s, const HalfWalkParams& p) {
  return LaunchWithLds(kernel, grid, block, lds, s, p);
}

template <int NR>
hipError_t ByTile(int tp, dim3 grid, dim3 block, size_t lds, hipStream_t s, const HalfWalkParams& p) {
  switch (tp) {
    case 128:
      return LaunchBig(HalfWalkKernel<NR, 128>, grid, block, lds, s, p);
    case 64:
      return LaunchBig(HalfWalkKernel<NR, 64>, grid, block, lds, s, p);
    case 32:
      return LaunchBig(HalfWalkKernel<NR, 32>, grid, block, lds, s, p);
    case 16:
      return LaunchBig(HalfWalkKernel<NR, 16>, grid, block, lds, s, p);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace

hipError_t LaunchHalfWalk(int nrows, int tile_pos, int threads, const HalfWalkParams& p, hipStream_t stream) {
  if (p.P == 0 || p.n_groups == 0) return hipSuccess;
  const size_t lds = (size_t)(p.K + 1) * tile_pos * 2;
  if (lds > (size_t)kMaxLdsBytes || threads < tile_pos || threads % 64 != 0 || p.slices < 1) return hipErrorInvalidValue;
  HalfWalkParams q = p;
  q.tiles = (int)((p.P + tile_pos - 1) / tile_pos);
  dim3 grid(8u * (uint32_t)q.slices * (((uint32_t)q.tiles + 7) / 8)), block(threads);
  return nrows == 2 ? ByTile<2>(tile_pos, grid, block, lds, stream, q) : ByTile<1>(tile_pos, grid, block, lds, stream, q);
}

template <int NR, int PPL>
hipError_t HalfChunkLaunch(const HalfChunkWalkParams& p, hipStream_t stream) {
  constexpr int kTile = 64 * PPL;
  HalfChunkWalkParams q = p;
  q.tiles = (int)((p.P + kTile - 1) / kTile);
  const size_t lds = (size_t)(kCChunk + 1) * kTile * 2;
  dim3 grid(8u * (uint32_t)q.slices * (((uint32_t)q.tiles + 7) / 8)), block(64 * kCWaves);
  auto kernel = HalfChunkWalkKernel<NR, kChunkWalkGroups, PPL>;
  return LaunchWithLds(kernel, grid, block, lds, stream, q);
}

// Needs hw % 4 == 0 and 8-byte aligned x / out.  Four positions per lane (256
// per workgroup); eight per lane halve the number of workgroups and measured
// 46.5 us against 28.1 us on the 256 -> 512 @28x28 configuration.
hipError_t LaunchHalfChunkWalk(int nrows, const HalfChunkWalkParams& p, hipStream_t stream) {
  if (p.P == 0 || p.n_groups == 0) return hipSuccess;
  if (p.hw % 4 != 0 || p.n_chunks < 1 || p.slices < 1) return hipErrorInvalidValue;
  return nrows == 2 ? HalfChunkLaunch<2, 4>(p, stream) : HalfChunkLaunch<1, 4>(p, stream);
}

// A lane's positions are one piece of one image: eight positions per lane need hw % 8 == 0 and 16-byte aligned
// x / out, four (the narrow form) hw % 4 == 0 and 8-byte alignment; with kTileWalkRagged any map size.
hipError_t LaunchHalfTileWalk(int nrows, const HalfTileWalkParams& p, hipStream_t stream) {
  if (p.P == 0 || p.n_groups == 0) return hipSuccess;
  const int form = p.form & (kTileWalkRagged - 1);
  const bool ragged = (p.form & kTileWalkRagged) != 0;
  if (form >= kHalfTileWalkForms) return hipErrorInvalidValue;
  const int tile = HalfTileWalkTileOf(form), ppl = form == kHalfTileWalkNarrowForm ? 4 : 8;
  if (!ragged && p.hw % ppl != 0) return hipErrorInvalidValue;
  const size_t lds = TileWalkLdsBytes(p.K, tile * 2);
  if (lds > (size_t)kMaxLdsBytes) return hipErrorInvalidValue;
  HalfTileWalkParams q = p;
  q.tiles = (int)((p.P + (uint32_t)tile - 1) / (uint32_t)tile);
  uint32_t slots = ((uint32_t)q.tiles + 7) / 8;  // workgroups per XCD
  if (q.split == 2) {
    if (q.parts < 2 || (int64_t)q.parts * slots > q.split_slots) return hipErrorInvalidValue;
    slots *= (uint32_t)q.parts;
  } else if (q.split != 0) {
    if (q.split_slots < (int)slots + 1) return hipErrorInvalidValue;  // every XCD needs a spare workgroup
    slots = (uint32_t)q.split_slots;
  }
  dim3 grid(8u * slots), block(64 * kTwWaves);
  const bool two = nrows == 2;
  switch (form) {
    case 0:
      return two ? LaunchWithHead(HalfTileWalkKernel<2, 2, 8>, grid, block, lds, stream, q) : LaunchWithHead(HalfTileWalkKernel<1, 2, 8>, grid, block, lds, stream, q);
    case 1:
      return two ? LaunchWithHead(HalfTileWalkKernel<2, 4, 8>, grid, block, lds, stream, q) : LaunchWithHead(HalfTileWalkKernel<1, 4, 8>, grid, block, lds, stream, q);
    case 2:
      return two ? LaunchWithHead(HalfTileWalkKernel<2, 8, 8>, grid, block, lds, stream, q) : LaunchWithHead(HalfTileWalkKernel<1, 8, 8>, grid, block, lds, stream, q);
    case 3:
      return two ? LaunchWithHead(HalfTileWalkKernel<2, 16, 8>, grid, block, lds, stream, q) : LaunchWithHead(HalfTileWalkKernel<1, 16, 8>, grid, block, lds, stream, q);
    default:  // the narrow form
      return two ? LaunchWithHead(HalfTileWalkKernel<2, 2, 4>, grid, block, lds, stream, q) : LaunchWithHead(HalfTileWalkKernel<1, 2, 4>, grid, block, lds, stream, q);
  }
}

}  // namespace pl
