// fp32 row walk over channel chunks.
//
// The plain row walk keeps all input channels of a tile in LDS, which limits
// a tile to 128 or 64 positions once there are a few hundred channels; every
// (tile, row) pair streams the row's index list through the scalar cache, and
// that stream is what bounds the kernel.  Here a workgroup (8 wavefronts)
// takes 256 positions and stages the channels kChunk at a time; a wavefront
// owns G row groups, keeps their accumulators in registers across the chunks
// and walks, per chunk, only the entries whose channel lies in it.  One list
// fetch then serves 256 positions whatever the channel count, entries carry
// an 8-bit chunk-local channel, and a lane works on four consecutive
// positions (one 16-byte LDS read per entry, 1 KB contiguous per store).
// The order of the fused multiply-adds of one output is the index order, as
// in the plain walk.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "epilogue.h"
#include "launch_lds.h"
#include "sparse_conv_kernels.h"

namespace pl {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(4))) uint32_t* ConstWords;
typedef const __attribute__((address_space(4))) float* ConstFloats;

using epilogue::ActivateT;

// Workgroup id -> tile: each XCD (linear id mod 8) owns a contiguous range of
// tiles, the per_tile workgroups of one tile follow each other on it.
__device__ __forceinline__ int XcdTile(int tiles, int per_tile) {
  const int xcd = blockIdx.x & 7, wg_slot = blockIdx.x >> 3;
  const int first = (xcd * tiles) >> 3, last = ((xcd + 1) * tiles) >> 3;
  const int t = first + wg_slot / per_tile;
  return t < last ? t : -1;
}

constexpr int kTile = kChunkWalkTile;    // positions per workgroup
constexpr int kChunk = kChunkWalkChunk;  // channels staged at once
constexpr int kWaves = kChunkWalkWaves;

template <int NR, int G, int ACT>
__device__ __forceinline__ void ChunkWalkBody(const ChunkWalkParams& p, uint32_t* tile) {
  const int tile_id = XcdTile(p.tiles, p.slices);
  if (tile_id < 0) return;
  const int slice = (blockIdx.x >> 3) % p.slices;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t tile0 = (uint32_t)tile_id * (uint32_t)kTile;

  const ConstWords group_words = (ConstWords)p.groups;
  const ConstFloats biasp = (ConstFloats)p.bias;
  const ConstWords descp = (ConstWords)p.desc;
  const ConstWords idxp = (ConstWords)p.idx;
  const ConstWords wtsp = (ConstWords)p.wts;

  // accumulators of the wavefront's G row groups start at the bias
  const int g_first = (slice * kWaves + wave) * G;
  float acc[G][NR][4];
#pragma unroll
  for (int gi = 0; gi < G; ++gi) {
    const int g = g_first + gi;
    float b0 = 0.0f, b1 = 0.0f;
    if (g < p.n_groups && biasp) {
      const int row0 = (int)group_words[(size_t)g * 4], nrows = (int)group_words[(size_t)g * 4 + 1];
      b0 = biasp[row0];
      if (NR == 2 && nrows == 2) b1 = biasp[row0 + 1];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[gi][0][j] = b0;
      if (NR == 2) acc[gi][NR - 1][j] = b1;
    }
  }

  // staging: thread = (four positions, channel row of a pass of 8 rows)
  const int j4 = tid & 63, r0 = tid >> 6;
  const uint32_t gpos = tile0 + 4u * (uint32_t)j4;
  const bool live = gpos < p.P;
  const uint32_t n = live ? gpos / (uint32_t)p.hw : 0u;
  const uint32_t pp = live ? gpos % (uint32_t)p.hw : 0u;
  const float* xcol = static_cast<const float*>(p.x) + (size_t)n * p.K * p.hw + pp;
  const uint32_t* xlane = tile + 4 * lane;  // the lane's four positions of LDS row 0

  // The next chunk travels from memory into registers while the current one
  // is walked (the walk itself issues no vector memory instruction, so it
  // never waits for these loads); the registers are written to LDS once every
  // wavefront has finished with the current chunk.
  uint4 v[kChunk / kWaves];
  auto fetch = [&](int chunk) {
    const int c0 = chunk * kChunk;
#pragma unroll
    for (int u = 0; u < kChunk / kWaves; ++u) {
      const int ch = min(c0 + r0 + kWaves * u, p.K - 1);
      v[u] = *reinterpret_cast<const uint4*>(xcol + (size_t)ch * p.hw);
    }
  };
  fetch(0);
  for (int chunk = 0; chunk < p.n_chunks; ++chunk) {
    if (chunk > 0) __syncthreads();  // the previous chunk is read until every wavefront has walked it
    {
      const int c0 = chunk * kChunk;
#pragma unroll
      for (int u = 0; u < kChunk / kWaves; ++u) {
        const int kl = r0 + kWaves * u;
        const bool on = live && c0 + kl < p.K;
        *reinterpret_cast<uint4*>(tile + (size_t)kl * kTile + 4 * j4) = on ? v[u] : make_uint4(0, 0, 0, 0);
      }
      // row kChunk is all zero: the target of list padding entries
      if (chunk == 0 && tid < kTile / 4) *reinterpret_cast<uint4*>(tile + (size_t)kChunk * kTile + 4 * tid) = make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
    if (chunk + 1 < p.n_chunks) fetch(chunk + 1);

    const ConstWords dw = descp + ((size_t)((slice * p.n_chunks + chunk) * kWaves + wave) * G) * 2;
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
      const uint32_t first = dw[2 * gi], entries = dw[2 * gi + 1];
      const ConstWords ip = idxp + first;
      const ConstWords wp = wtsp + (size_t)first * (4 * NR);
      auto entry = [&](uint32_t kl, uint32_t w0, uint32_t w1) {
        const uint4 xv = *reinterpret_cast<const uint4*>(xlane + (size_t)kl * kTile);
        const float x4[4] = {__uint_as_float(xv.x), __uint_as_float(xv.y), __uint_as_float(xv.z), __uint_as_float(xv.w)};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[gi][0][j] = __builtin_fmaf(x4[j], __uint_as_float(w0), acc[gi][0][j]);
          if (NR == 2) acc[gi][NR - 1][j] = __builtin_fmaf(x4[j], __uint_as_float(w1), acc[gi][NR - 1][j]);
        }
      };
      const uint32_t batches = entries >> 2, rem = entries & 3u;
      for (uint32_t b = 0; b < batches; ++b) {
        const uint32_t packed = ip[b];
        uint32_t w[4 * NR];
#pragma unroll
        for (int i = 0; i < 4 * NR; ++i) w[i] = wp[(size_t)b * (4 * NR) + i];
#pragma unroll
        for (int e = 0; e < 4; ++e) entry((packed >> (8 * e)) & 0xffu, w[e * NR], w[e * NR + NR - 1]);
      }
      if (rem != 0) {  // the last, partly filled batch: only its real entries
        const uint32_t packed = ip[batches];
        uint32_t w[3 * NR];
#pragma unroll
        for (int i = 0; i < 3 * NR; ++i) w[i] = wp[(size_t)batches * (4 * NR) + i];
        entry(packed & 0xffu, w[0], w[NR - 1]);
        if (rem > 1) entry((packed >> 8) & 0xffu, w[NR], w[NR + NR - 1]);
        if (rem > 2) entry((packed >> 16) & 0xffu, w[2 * NR], w[2 * NR + NR - 1]);
      }
    }
  }

  // epilogue: the lane's four positions of every row of its groups
  const uint32_t opos = tile0 + 4u * (uint32_t)lane;
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
        v4f o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = ActivateT<ACT>(acc[gi][r][j], p.act);
        float* dst = static_cast<float*>(p.out) + ((size_t)on * p.M + row0 + r) * p.hw + opp;
        __builtin_nontemporal_store(o, reinterpret_cast<v4f*>(dst));
      }
    }
  }
}

template <int NR, int G>
__global__ void __launch_bounds__(64 * kChunkWalkWaves, 2) ChunkWalkKernel(const ChunkWalkParams p) {
  extern __shared__ uint32_t tile[];
  switch (p.act.type) {
    case 1:
      ChunkWalkBody<NR, G, 1>(p, tile);
      break;
    case 2:
      ChunkWalkBody<NR, G, 2>(p, tile);
      break;
    case 4:
      ChunkWalkBody<NR, G, 4>(p, tile);
      break;
    case 10:
      ChunkWalkBody<NR, G, 10>(p, tile);
      break;
    default:
      ChunkWalkBody<NR, G, 0>(p, tile);
      break;
  }
}

template <typename K>
hipError_t LaunchBig(K kernel, dim3 grid, dim3 block, size_t lds, hipStream_t s, const ChunkWalkParams& p) {
  return LaunchWithLds(kernel, grid, block, lds, s, p);
}

}  // namespace

hipError_t LaunchChunkWalk(int nrows, const ChunkWalkParams& p, hipStream_t stream) {
  if (p.P == 0 || p.n_groups == 0) return hipSuccess;
  if (p.hw % 4 != 0 || p.n_chunks < 1 || p.slices < 1 || (p.groups_per_wave != 4 && p.groups_per_wave != 8)) return hipErrorInvalidValue;
  ChunkWalkParams q = p;
  q.tiles = (int)((p.P + kTile - 1) / kTile);
  const size_t lds = (size_t)(kChunk + 1) * kTile * 4;
  dim3 grid(8u * (uint32_t)q.slices * (((uint32_t)q.tiles + 7) / 8)), block(64 * kWaves);
  if (p.groups_per_wave == 4) {
    if (nrows == 2) return LaunchBig(ChunkWalkKernel<2, 4>, grid, block, lds, stream, q);
    return LaunchBig(ChunkWalkKernel<1, 4>, grid, block, lds, stream, q);
  }
  if (nrows == 2) return LaunchBig(ChunkWalkKernel<2, 8>, grid, block, lds, stream, q);
  return LaunchBig(ChunkWalkKernel<1, 8>, grid, block, lds, stream, q);
}

}  // namespace pl
