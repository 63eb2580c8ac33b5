// gfx950 kernels of the sparse 1x1 convolution (sparse weights x dense
// activations).  Two algorithms:
//
//  * row walk  - a workgroup stages a tile of activation positions in LDS
//                ([channel][position] dwords; int8 channels packed four to a
//                dword), every wavefront owns one output row (or a pair that
//                shares indices) at a time and walks that row's nonzero list
//                once.  fp32 accumulates with fmaf in index order starting
//                from the bias, exactly the order of the reference's math
//                functions (lite/backends/arm/math/sparse_conv_impl.cc:27-216);
//                int8 accumulates exactly in int32 with v_dot4.
//  * block MFMA - int8 only: the weight matrix is cut into 32x32 blocks, the
//                blocks holding a nonzero are multiplied on the matrix cores
//                (v_mfma_i32_32x32x32_i8), empty blocks are skipped.  A
//                wavefront keeps its 32 output rows' blocks in registers and
//                streams 128 activation positions through them.
//
// Both end in the same epilogue: v = fmaf(float(acc), scale, bias), the
// activation, then fp32 store or int8 requantisation (max(v,-127), round half
// away from zero, saturate), as in sparse_conv_impl.cc:1661-1685, :3633-3643.
//
// Positions are the flattened (image, pixel) index g = n*hw + p, so tiles do
// not care about image boundaries.
#include "epilogue.h"
#include "launch_lds.h"
#include "sparse_conv_kernels.h"

#include <type_traits>

// This file is compiled as four translation units (in parallel) selected by
// PL_KERNEL_PART: 0 = row walk + launch selection, 1 / 2 / 3 = block MFMA
// kernels with fp32 / int8 / int32 output.  Without the macro everything is
// built in one unit.
#ifndef PL_KERNEL_PART
#define PL_PART_WALK 1
#define PL_PART_MFMA_F32 1
#define PL_PART_MFMA_I8 1
#define PL_PART_MFMA_ACC32 1
#else
#define PL_PART_WALK (PL_KERNEL_PART == 0)
#define PL_PART_MFMA_F32 (PL_KERNEL_PART == 1)
#define PL_PART_MFMA_I8 (PL_KERNEL_PART == 2)
#define PL_PART_MFMA_ACC32 (PL_KERNEL_PART == 3)
#endif
#define PL_PART_MFMA_ANY (PL_PART_MFMA_F32 || PL_PART_MFMA_I8 || PL_PART_MFMA_ACC32)

namespace pl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// Outputs are written once and never read back by the kernel: store them
// non-temporally so that they stream to memory instead of sitting dirty in
// L2 until the end-of-kernel write-back.
__device__ __forceinline__ void StreamStore(float4 v, void* dst) {
  __builtin_nontemporal_store(v4f{v.x, v.y, v.z, v.w}, static_cast<v4f*>(dst));
}
__device__ __forceinline__ void StreamStore(int4 v, void* dst) {
  __builtin_nontemporal_store(v4i{v.x, v.y, v.z, v.w}, static_cast<v4i*>(dst));
}
__device__ __forceinline__ void StreamStore(uint32_t v, void* dst) { __builtin_nontemporal_store(v, static_cast<uint32_t*>(dst)); }
__device__ __forceinline__ void StreamStore(uint16_t v, void* dst) { __builtin_nontemporal_store(v, static_cast<uint16_t*>(dst)); }
__device__ __forceinline__ void StreamStore(float2 v, void* dst) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  __builtin_nontemporal_store(v2f{v.x, v.y}, static_cast<v2f*>(dst));
}
__device__ __forceinline__ void StreamStore(int2 v, void* dst) {
  typedef int v2i __attribute__((ext_vector_type(2)));
  __builtin_nontemporal_store(v2i{v.x, v.y}, static_cast<v2i*>(dst));
}

// Workgroups are handed to the 8 XCDs round robin (linear id mod 8).  For a
// 1-D grid of 8 * per_tile * ceil(tiles / 8) workgroups, the tile of this
// workgroup: XCD x owns the contiguous tiles [x*tiles/8, (x+1)*tiles/8), and
// the per_tile workgroups of one tile follow each other on that XCD.
// Returns -1 for the surplus workgroups of an XCD with the smaller share.
__device__ __forceinline__ int XcdTile(int tiles, int per_tile) {
  const int xcd = blockIdx.x & 7, wg_slot = blockIdx.x >> 3;
  const int first = (xcd * tiles) >> 3, last = ((xcd + 1) * tiles) >> 3;
  const int t = first + wg_slot / per_tile;
  return t < last ? t : -1;
}

// ---------------------------------------------------------------- epilogue
using namespace epilogue;  // activation, quantisation, packing (epilogue.h)

// 4x4 byte transpose: r[i] holds bytes (i, 0..3); on return r[j] holds bytes
// (0..3, j).
__device__ __forceinline__ void Transpose4x4(uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3) {
  // perm(hi, lo, sel): selector bytes 0-3 pick from lo, 4-7 from hi
  uint32_t a = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
  uint32_t b = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
  uint32_t c = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
  uint32_t d = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
  r0 = __builtin_amdgcn_perm(c, a, 0x05040100u);  // a.b0 a.b1 c.b0 c.b1
  r1 = __builtin_amdgcn_perm(c, a, 0x07060302u);
  r2 = __builtin_amdgcn_perm(d, b, 0x05040100u);
  r3 = __builtin_amdgcn_perm(d, b, 0x07060302u);
}

// ------------------------------------------------------------ tile staging
// fp32: tile[k][TP] floats plus one row of zeros.  int8: tile[q][TP] dwords, dword = channels
// 4q..4q+3 of one position (channels past K read as zero).  The aligned path
// issues a batch of row loads before it touches LDS so that they are in
// flight together.
template <bool INT8, int TP>
__device__ __forceinline__ void StageTile(uint32_t* tile, const WalkParams& p, uint32_t tile0) {
  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  // fp32 tiles end in an all-zero row, the target of list padding entries
  if (!INT8 && tid < TP) tile[(size_t)p.kd * TP + tid] = 0u;
  if (p.vec) {
    constexpr int TPV = TP / 4;  // groups of four positions per row
    const int j4 = tid % TPV;
    const uint32_t g = tile0 + 4u * j4;
    const bool live = g < p.P;
    const uint32_t n = live ? g / (uint32_t)p.hw : 0u;
    const uint32_t pp = live ? g % (uint32_t)p.hw : 0u;
    const int k_step = nthreads / TPV;
    if (!INT8) {
      constexpr int kBatch = 8;
      const float* base = static_cast<const float*>(p.x) + (size_t)n * p.K * p.hw + pp;
      for (int k0 = tid / TPV; k0 < p.kd; k0 += kBatch * k_step) {
        uint4 v[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int k = min(k0 + u * k_step, p.kd - 1);
          v[u] = *reinterpret_cast<const uint4*>(base + (size_t)k * p.hw);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int k = k0 + u * k_step;
          if (k < p.kd) *reinterpret_cast<uint4*>(tile + (size_t)k * TP + 4 * j4) = live ? v[u] : make_uint4(0, 0, 0, 0);
        }
      }
    } else {
      constexpr int kBatch = 4;
      const int8_t* base = static_cast<const int8_t*>(p.x) + (size_t)n * p.K * p.hw + pp;
      for (int k0 = tid / TPV; k0 < p.kd; k0 += kBatch * k_step) {
        uint32_t r[kBatch][4];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int k = min(k0 + u * k_step, p.kd - 1);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int ch = min(4 * k + i, p.K - 1);
            r[u][i] = *reinterpret_cast<const uint32_t*>(base + (size_t)ch * p.hw);
          }
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int k = k0 + u * k_step;
#pragma unroll
          for (int i = 0; i < 4; ++i) r[u][i] = (live && 4 * k + i < p.K) ? r[u][i] : 0u;
          Transpose4x4(r[u][0], r[u][1], r[u][2], r[u][3]);
          if (k < p.kd) *reinterpret_cast<uint4*>(tile + (size_t)k * TP + 4 * j4) = make_uint4(r[u][0], r[u][1], r[u][2], r[u][3]);
        }
      }
    }
  } else {
    const int j = tid % TP;
    const uint32_t g = tile0 + j;
    const bool live = g < p.P;
    const uint32_t n = live ? g / (uint32_t)p.hw : 0u;
    const uint32_t pp = live ? g % (uint32_t)p.hw : 0u;
    for (int k = tid / TP; k < p.kd; k += nthreads / TP) {
      uint32_t v = 0;
      if (live) {
        if (!INT8) {
          v = __float_as_uint(static_cast<const float*>(p.x)[((size_t)n * p.K + k) * p.hw + pp]);
        } else {
          const int8_t* src = static_cast<const int8_t*>(p.x) + ((size_t)n * p.K + 4 * k) * p.hw + pp;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            uint32_t b = (4 * k + i < p.K) ? (uint32_t)(uint8_t)src[(size_t)i * p.hw] : 0u;
            v |= b << (8 * i);
          }
        }
      }
      tile[(size_t)k * TP + j] = v;
    }
  }
}

// ------------------------------------------------------------------ stores
template <int OUT>
__device__ __forceinline__ void StoreOne(void* out, size_t idx, float v, int acc) {
  if (OUT == kOutF32) {
    static_cast<float*>(out)[idx] = v;
  } else if (OUT == kOutI8) {
    static_cast<int8_t*>(out)[idx] = static_cast<int8_t>(QuantizeI8(v));
  } else {
    static_cast<int*>(out)[idx] = acc;
  }
}

// Store PPL consecutive positions of one output row.  `g` is the first
// position; with vec the PPL positions lie in one image and are aligned.
template <int OUT, int PPL>
__device__ __forceinline__ void StoreRow(const WalkParams& p, int row, uint32_t g, const float* v, const int* acc) {
  if (g >= p.P) return;
  if (p.vec) {
    const uint32_t n = g / (uint32_t)p.hw, pp = g % (uint32_t)p.hw;
    const size_t idx = ((size_t)n * p.M + row) * p.hw + pp;
    if (OUT == kOutF32) {
      float* dst = static_cast<float*>(p.out) + idx;
      if (PPL == 4) {
        StreamStore(make_float4(v[0], v[1], v[2], v[3]), dst);
      } else if (PPL == 2) {
        StreamStore(make_float2(v[0], v[1]), dst);
      } else {
        __builtin_nontemporal_store(v[0], dst);
      }
    } else if (OUT == kOutI8) {
      int8_t* dst = static_cast<int8_t*>(p.out) + idx;
      if (PPL == 4) {
        StreamStore(TruncPackI8x4(QuantizeF(v[0]), QuantizeF(v[1]), QuantizeF(v[2]), QuantizeF(v[3])), dst);
      } else {
#pragma unroll
        for (int j = 0; j < PPL; ++j) dst[j] = static_cast<int8_t>(QuantizeI8(v[j]));
      }
    } else {
      int* dst = static_cast<int*>(p.out) + idx;
#pragma unroll
      for (int j = 0; j < PPL; ++j) dst[j] = acc[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < PPL; ++j) {
      const uint32_t gj = g + j;
      if (gj < p.P) {
        const uint32_t n = gj / (uint32_t)p.hw, pp = gj % (uint32_t)p.hw;
        StoreOne<OUT>(p.out, ((size_t)n * p.M + row) * p.hw + pp, v[j], acc[j]);
      }
    }
  }
}

// ---------------------------------------------------------------- row walk
#if PL_PART_WALK
// Multiply-accumulate of one index entry into the lane's PPL positions.
template <bool INT8, int NR, int PPL, int TP>
__device__ __forceinline__ void WalkEntry(const uint32_t* xbase, uint32_t k, uint32_t w0, uint32_t w1, float (&f0)[PPL], float (&f1)[PPL], int (&a0)[PPL], int (&a1)[PPL]) {
  const uint32_t* xp = xbase + (size_t)k * TP;
  uint32_t xv[PPL];
  if (PPL == 4) {
    uint4 t = *reinterpret_cast<const uint4*>(xp);
    xv[0] = t.x;
    xv[1 % PPL] = t.y;
    xv[2 % PPL] = t.z;
    xv[3 % PPL] = t.w;
  } else if (PPL == 2) {
    uint2 t = *reinterpret_cast<const uint2*>(xp);
    xv[0] = t.x;
    xv[1 % PPL] = t.y;
  } else {
    xv[0] = xp[0];
  }
#pragma unroll
  for (int j = 0; j < PPL; ++j) {
    if (INT8) {
      a0[j] = __builtin_amdgcn_sdot4((int)xv[j], (int)w0, a0[j], false);
      if (NR == 2) a1[j] = __builtin_amdgcn_sdot4((int)xv[j], (int)w1, a1[j], false);
    } else {
      f0[j] = __builtin_fmaf(__uint_as_float(xv[j]), __uint_as_float(w0), f0[j]);
      if (NR == 2) f1[j] = __builtin_fmaf(__uint_as_float(xv[j]), __uint_as_float(w1), f1[j]);
    }
  }
}

template <bool INT8, int OUT, int NR, int TP, int ACT>
__device__ __forceinline__ void RowWalkBody(const WalkParams& p, uint32_t* tile) {
  constexpr int PPL = TP >= 64 ? TP / 64 : 1;  // positions per lane
  // Index lists, weights, scales and biases are wave-uniform and written by
  // the host before the launch: read them through the constant address
  // space, i.e. with scalar loads.  Left to itself the compiler turns some
  // of them into vector loads of one address per wavefront, which cost a
  // full address-coalescing pass each and, for the bias, make the walk wait
  // for the previous row's output stores.
  typedef const __attribute__((address_space(4))) float* ConstFloats;
  typedef const __attribute__((address_space(4))) uint32_t* ConstWords;
  const ConstFloats biasp = (ConstFloats)p.bias;
  const ConstFloats scalep = (ConstFloats)p.scale;
  static_assert(sizeof(DevGroup) == 16, "DevGroup is read as four words");
  const ConstWords group_words = (ConstWords)p.groups;
  // 1-D grid; the slices (row ranges) of one tile are neighbours in the
  // per-XCD order so that the tile is fetched into one L2
  const int tile_id = XcdTile(p.tiles, p.slices);
  const int slice = (blockIdx.x >> 3) % p.slices;
  if (tile_id < 0) return;
  const uint32_t tile0 = (uint32_t)tile_id * (uint32_t)TP;
  StageTile<INT8, TP>(tile, p, tile0);
  __syncthreads();

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nwaves = blockDim.x >> 6;
  const int g_begin = slice * p.groups_per_slice;
  const int g_end = min(p.n_groups, g_begin + p.groups_per_slice);
  const bool lane_on = (TP >= 64) || (lane < TP);
  const uint32_t* xbase = tile + (lane_on ? lane * PPL : 0);

  for (int g = g_begin + wave; g < g_end; g += nwaves) {
    const ConstWords gw = group_words + (size_t)g * 4;
    const DevGroup grp = {(int)gw[0], (int)gw[1], gw[2], gw[3]};
    const ConstWords kp = (ConstWords)p.kidx + grp.first;
    const ConstWords wp = (ConstWords)p.wts + (size_t)grp.first * NR;

    float f0[PPL], f1[PPL];
    int a0[PPL], a1[PPL];
#pragma unroll
    for (int j = 0; j < PPL; ++j) {
      a0[j] = a1[j] = 0;
      f0[j] = f1[j] = 0.0f;
    }
    if (!INT8) {
      // the accumulator starts at the bias, entries follow in index order
      const float b0 = biasp ? biasp[grp.row0] : 0.0f;
      const float b1 = (biasp && NR == 2 && grp.nrows == 2) ? biasp[grp.row0 + 1] : 0.0f;
#pragma unroll
      for (int j = 0; j < PPL; ++j) {
        f0[j] = b0;
        f1[j] = b1;
      }
    }

    // the list length is a multiple of kWalkBatch: no remainder loop, whose
    // entries would each wait for their own scalar loads
    for (uint32_t e = 0; e < grp.count; e += kWalkBatch) {
#pragma unroll
      for (int j = 0; j < kWalkBatch; ++j)
        WalkEntry<INT8, NR, PPL, TP>(xbase, kp[e + j], wp[(size_t)(e + j) * NR], NR == 2 ? wp[(size_t)(e + j) * NR + NR - 1] : 0u, f0, f1, a0, a1);
    }

    if (!lane_on) continue;
    const uint32_t gpos = tile0 + (uint32_t)lane * PPL;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (r == 1 && grp.nrows < 2) break;
      const int row = grp.row0 + r;
      float v[PPL];
      const int* acc = r == 0 ? a0 : a1;
      if (INT8) {
        if (OUT != kOutAcc32) {
          const float s = scalep[row];
          const float b = biasp ? biasp[row] : 0.0f;
#pragma unroll
          for (int j = 0; j < PPL; ++j) v[j] = ActivateT<ACT>(__builtin_fmaf((float)acc[j], s, b), p.act);
        }
      } else {
        const float* f = r == 0 ? f0 : f1;
#pragma unroll
        for (int j = 0; j < PPL; ++j) v[j] = ActivateT<ACT>(f[j], p.act);
      }
      StoreRow<OUT, PPL>(p, row, gpos, v, acc);
    }
  }
}

template <bool INT8, int OUT, int NR, int TP>
__global__ void __launch_bounds__(1024) RowWalkKernel(const WalkParams p) {
  extern __shared__ uint32_t tile[];
  DispatchAct(OUT == kOutAcc32 ? 0 : p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    RowWalkBody<INT8, OUT, NR, TP, ACT>(p, tile);
  });
}
#endif  // PL_PART_WALK

// -------------------------------------------------------------- block MFMA
#if PL_PART_MFMA_ANY
// Positions are handled four at a time ("quads").  Every image is cut into
// qpi = ceil(hw / 4) quads, so a quad never leaves its image; when hw is not
// a multiple of four the last quad of an image holds hw % 4 valid positions.
// Quads of all images form one sequence (index n*qpi + q); a workgroup
// (4 wavefronts = 4 blocks of 32 output rows) handles a tile of J <= 32
// consecutive quads.  MFMA column j of accumulator c is position c of the
// tile's quad j, so a lane ends up with the four consecutive positions of
// each of its rows (one 16-byte fp32 store or one dword int8 store).
// LDS: xt[kg][c*32 + j], 16-byte cells, kg = group of 16 input channels.
struct QuadInfo {
  uint32_t n;    // image
  uint32_t pp;   // first position of the quad in its image
  int valid;     // 0: beyond the last image; else positions in the quad (1..4)
};

__device__ __forceinline__ QuadInfo LocateQuad(const MfmaParams& p, uint32_t quad) {
  QuadInfo q;
  const bool live = quad < p.total_quads;
  const uint32_t qs = live ? quad : 0u;
  q.n = qs / (uint32_t)p.qpi;
  q.pp = 4u * (qs - q.n * (uint32_t)p.qpi);
  const int left = p.hw - (int)q.pp;
  q.valid = !live ? 0 : (left < 4 ? left : 4);
  return q;
}

// Issue the dword loads of one channel group for one quad.  Global memory
// needs no alignment for dword access.  A partial quad (valid < 4) reads the
// last four positions of its row (CommitX shifts the unwanted ones out), so
// no load leaves the tensor.  All loads are unconditional so that they are in
// flight together.  FAST: the channel groups are complete and the tensor is
// below 2 GB, so an address is a uniform base plus one 32-bit per-lane offset
// (no per-load address arithmetic on the vector ALU).  Otherwise channel
// indices are clamped and the values masked in CommitX.  Lanes beyond the
// last image read the tensor's first bytes and are ignored.
template <bool FAST>
__device__ __forceinline__ void LoadX(uint32_t (&r)[16], const MfmaParams& p, const QuadInfo& q, int kg_base, int kg_lane) {
  const bool live = q.valid > 0;
  const uint32_t first = (q.valid == 4 || !live) ? q.pp : (uint32_t)(p.hw - 4);  // hw >= 4 on this path
  if (FAST) {
    const uint32_t voff = live ? (q.n * (uint32_t)p.K + 16u * (uint32_t)kg_lane) * (uint32_t)p.hw + first : 0u;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int8_t* sbase = p.x + (size_t)(16 * kg_base + i) * (size_t)p.hw;  // uniform
      r[i] = *reinterpret_cast<const uint32_t*>(sbase + voff);
    }
  } else {
    const int8_t* col = p.x + (live ? (size_t)q.n * p.K * p.hw + first : (size_t)0);
    const size_t row_step = live ? (size_t)p.hw : (size_t)0;
    const int kg = kg_base + kg_lane;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int ch = min(16 * kg + i, p.K - 1);
      r[i] = *reinterpret_cast<const uint32_t*>(col + (size_t)ch * row_step);
    }
  }
}

// Transpose to channel-innermost and write the cells of four positions.
template <bool FAST>
__device__ __forceinline__ void CommitX(uint32_t (&r)[16], uint4* xt, const MfmaParams& p, const QuadInfo& q, bool live, bool store, int kg_base, int kg_lane, int j, int kg_lds0 = 0) {
  const int n_kg = 2 * p.ksteps;
  const int kg = kg_base + kg_lane;  // kg_lds0: the channel group held by LDS row 0
  if (!p.quad_aligned) {
    // a partial quad was read from the last four positions of its row
    const int sh = (q.valid == 4 || q.valid == 0) ? 0 : 8 * (4 - q.valid);
#pragma unroll
    for (int i = 0; i < 16; ++i) r[i] >>= sh;
  }
  if (!FAST) {
#pragma unroll
    for (int i = 0; i < 16; ++i) r[i] = (live && 16 * kg + i < p.K) ? r[i] : 0u;
  }
#pragma unroll
  for (int b = 0; b < 4; ++b) Transpose4x4(r[4 * b], r[4 * b + 1], r[4 * b + 2], r[4 * b + 3]);
  // now r[4b + c] = channels 16kg+4b..+3 of the quad's position c
  if (store && (FAST || kg < n_kg)) {
#pragma unroll
    for (int c = 0; c < 4; ++c) xt[(size_t)(kg - kg_lds0) * kMfmaTilePos + c * 32 + j] = make_uint4(r[c], r[4 + c], r[8 + c], r[12 + c]);
  }
}

// hw < 4: byte loads, one position at a time.  Stages the channel groups
// [kg_first, kg_end) into LDS rows 0 .. kg_end - kg_first.
__device__ __forceinline__ void StageMfmaBytes(uint4* xt, const MfmaParams& p, uint32_t quad, bool quad_on, int kg0, int j, int kg_first, int kg_end) {
  if (!quad_on) return;
  const QuadInfo q = LocateQuad(p, quad);
  for (int kg = kg_first + kg0; kg < kg_end; kg += 8) {
    for (int c = 0; c < 4; ++c) {
      uint32_t d[4] = {0, 0, 0, 0};
      if (c < q.valid) {
        const int8_t* col = p.x + (size_t)q.n * p.K * p.hw + q.pp + c;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int ch = 16 * kg + i;
          const uint32_t b = (ch < p.K) ? (uint32_t)(uint8_t)col[(size_t)ch * p.hw] : 0u;
          d[i >> 2] |= b << (8 * (i & 3));
        }
      }
      xt[(size_t)(kg - kg_first) * kMfmaTilePos + c * 32 + j] = make_uint4(d[0], d[1], d[2], d[3]);
    }
  }
}

template <int OUT>
__device__ __forceinline__ void StoreRun4(void* dst, const float* v, const int* q) {
  if (OUT == kOutF32) {
    StreamStore(make_float4(v[0], v[1], v[2], v[3]), dst);
  } else if (OUT == kOutI8) {
    StreamStore(PackI8x4(q[0], q[1], q[2], q[3]), dst);  // already quantised
  } else {
    StreamStore(make_int4(q[0], q[1], q[2], q[3]), dst);
  }
}

// ACT < 0: activation type read at run time (slow paths only).
template <int ACT>
__device__ __forceinline__ float ActivateAny(float v, const DevAct& a) {
  if (ACT < 0) return Activate(v, a);
  return ActivateT<(ACT < 0 ? 0 : ACT)>(v, a);
}

// Scales and biases of the 16 output rows a lane finishes (row
// 8*(r/4) + 4*(lane/32) + r%4 of the wavefront's row block), fetched ahead of
// the multiply so that the epilogue does not start with a memory wait.
struct RowConsts {
  float s[16], b[16];
};

template <int OUT>
__device__ __forceinline__ void LoadRowConsts(RowConsts& rc, const MfmaParams& p, int rb, int lane) {
  if (OUT == kOutAcc32) return;
  const int row_base = rb * 32 + 4 * (lane >> 5);
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    // four consecutive rows: one 16-byte load each (arrays are padded to 32 * row_blocks)
    const float4 sv = *reinterpret_cast<const float4*>(p.scale + row_base + 8 * g);
    const float4 bv = *reinterpret_cast<const float4*>(p.bias + row_base + 8 * g);
    rc.s[4 * g] = sv.x, rc.s[4 * g + 1] = sv.y, rc.s[4 * g + 2] = sv.z, rc.s[4 * g + 3] = sv.w;
    rc.b[4 * g] = bv.x, rc.b[4 * g + 1] = bv.y, rc.b[4 * g + 2] = bv.z, rc.b[4 * g + 3] = bv.w;
  }
}

// int8 output of a full tile inside one image: the wavefront's 32 rows x 128
// positions are packed, written to its own 4 KB of LDS as [row][128 bytes]
// and stored as 16 bytes per lane (8 rows x 128 contiguous bytes per
// instruction) instead of one dword per lane.  `stage` is private to the
// wavefront.
template <int ACT>
__device__ __forceinline__ void MfmaEpilogueI8Wide(const MfmaParams& p, const v16i (&acc)[4], const RowConsts& rc, int rb, int lane, uint32_t n, uint32_t pp, uint32_t* stage) {
  const int row_base = rb * 32 + 4 * (lane >> 5);
  const int j = lane & 31;
#pragma unroll
  for (int r = 0; r < 16; r += 2) {  // two rows at a time: their bytes are packed by the conversions themselves
    float f[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float s = rc.s[r + h], b = rc.b[r + h];
#pragma unroll
      for (int c = 0; c < 4; ++c) f[h][c] = ActQuantF<ACT>(__builtin_fmaf((float)acc[c][r + h], s, b), p.act);
    }
    uint32_t w0, w1;
    TruncPackI8x8(f[0][0], f[0][1], f[0][2], f[0][3], f[1][0], f[1][1], f[1][2], f[1][3], w0, w1);
    const int ro = 8 * (r >> 2) + (r & 3);  // r is even: row r + 1 is ro + 1
    stage[(4 * (lane >> 5) + ro) * 32 + j] = w0;  // row-local index 0..31, 32 dwords per row
    stage[(4 * (lane >> 5) + ro + 1) * 32 + j] = w1;
  }
  // the same wavefront reads back: its LDS operations complete in order
  char* obase = static_cast<char*>(p.out) + ((size_t)n * p.M + (size_t)rb * 32) * p.hw + pp;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 8 * i + (lane >> 3), chunk = lane & 7;
    const uint4 v = *reinterpret_cast<const uint4*>(stage + row * 32 + chunk * 4);
    StreamStore(make_int4((int)v.x, (int)v.y, (int)v.z, (int)v.w), obase + (size_t)row * p.hw + chunk * 16);
  }
}

// Accumulator register r of lane l is output row 8*(r/4) + 4*(l/32) + r%4 of
// the 32-row block, column l%32; the four accumulators are the positions of
// the lane's quad.  WHOLE: the quad has all four positions and the row block
// all 32 rows (the common case, kept free of per-row conditions).
template <int OUT, int ACT, bool WHOLE>
__device__ __forceinline__ void MfmaEpilogueRows(const MfmaParams& p, const v16i (&acc)[4], const RowConsts& rc, int row_base, char* lane_base, int valid) {
  constexpr uint32_t kElem = OUT == kOutI8 ? 1u : 4u;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int ro = 8 * (r >> 2) + (r & 3);
    if (!WHOLE && row_base + ro >= p.M) continue;
    char* dst = lane_base + (size_t)ro * (size_t)p.hw * kElem;
    int q[4];
    float v[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) q[c] = acc[c][r];
    if (OUT != kOutAcc32) {
      const float s = rc.s[r], b = rc.b[r];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float t = __builtin_fmaf((float)q[c], s, b);
        if (OUT == kOutI8) {
          q[c] = ActQuantI8<ACT>(t, p.act);  // from here on q holds the output bytes
        } else {
          v[c] = ActivateAny<ACT>(t, p.act);
        }
      }
    }
    if (WHOLE) {
      StoreRun4<OUT>(dst, v, q);
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (c < valid) {
          if (OUT == kOutF32) {
            reinterpret_cast<float*>(dst)[c] = v[c];
          } else if (OUT == kOutI8) {
            reinterpret_cast<int8_t*>(dst)[c] = static_cast<int8_t>(q[c]);
          } else {
            reinterpret_cast<int*>(dst)[c] = q[c];
          }
        }
      }
    }
  }
}

template <int OUT, int ACT>
__device__ __forceinline__ void MfmaEpilogue(const MfmaParams& p, const v16i (&acc)[4], const RowConsts& rc, int rb, int lane, const QuadInfo& qi) {
  if (qi.valid == 0) return;
  const int row_base = rb * 32 + 4 * (lane >> 5);
  constexpr uint32_t kElem = OUT == kOutI8 ? 1u : 4u;
  // per-lane part of the address; with a tensor below 2 GB it fits 32 bits
  // and rows are reached through a uniform base
  const size_t lane_off = (((size_t)qi.n * p.M + row_base) * p.hw + qi.pp) * kElem;
  char* lane_base = p.small ? static_cast<char*>(p.out) + (uint32_t)lane_off : static_cast<char*>(p.out) + lane_off;
  if (rb * 32 + 32 <= p.M && (p.quad_aligned || qi.valid == 4)) {
    MfmaEpilogueRows<OUT, ACT, true>(p, acc, rc, row_base, lane_base, 4);
  } else {
    MfmaEpilogueRows<OUT, ACT, false>(p, acc, rc, row_base, lane_base, qi.valid);
  }
}

// Epilogue of one (tile, row block) pair.  `stage` is the workgroup's LDS
// behind the activation tiles (4 KB per wavefront when p.i8_stage is set).
template <int OUT, int ACT, bool VEC>
__device__ __forceinline__ void MfmaFinish(const MfmaParams& p, uint32_t* stage, const v16i (&acc)[4], const RowConsts& rc, int rb, int lane, uint32_t quad0, int J) {
  if ((lane & 31) >= J) return;
  const QuadInfo qo = LocateQuad(p, quad0 + (uint32_t)(lane & 31));
  if (OUT == kOutI8 && VEC) {
    // wide stores need a full tile inside one image whose rows all exist and
    // 16-byte aligned row pieces
    const QuadInfo q0 = LocateQuad(p, quad0);
    const bool wide = p.i8_stage && J == 32 && p.small && rb * 32 + 32 <= p.M && (p.hw & 15) == 0 && quad0 + 32u <= p.total_quads && q0.pp + 128u <= (uint32_t)p.hw;
    if (wide) {
      MfmaEpilogueI8Wide<ACT>(p, acc, rc, rb, lane, q0.n, q0.pp, stage + (threadIdx.x >> 6) * 1024);
      return;
    }
  }
  MfmaEpilogue<OUT, ACT>(p, acc, rc, rb, lane, qo);
}

// One tile: stage, multiply, finish, pipelined over groups of four k-steps
// (activation loads feed the longest chain: transpose, LDS, barrier; the
// wavefront's weight blocks of the same k-steps follow right behind them).
template <int KSMAX, int OUT, int ACT, bool VEC>
__device__ __forceinline__ void MfmaTile(const MfmaParams& p, uint4* xt, uint32_t kmask, int rb, int rbc, bool wave_on, int tile) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int J = p.tile_quads;
  const int j = tid & 31;    // quad of the tile
  const int kg0 = tid >> 5;  // 8 channel groups per pass of the workgroup
  const uint32_t quad0 = (uint32_t)tile * (uint32_t)J;
  // KSMAX > 32 stands for any number of k-steps, taken kLoopChunk at a time
  // through one LDS tile; the accumulators stay in registers across chunks.
  constexpr bool kLoopK = KSMAX > 32;
  constexpr int KC = kLoopK ? kLoopChunk : KSMAX;  // k-steps held at once
  v4i a[KC];
  // Held across the multiply only by the 16-k-step kernel: the smaller ones
  // would lose a resident wavefront per SIMD to the 32 extra registers, the
  // 32-k-step one has no room left.
  constexpr bool kEarlyConsts = KSMAX == 16;
  RowConsts rc;
  if (kEarlyConsts) LoadRowConsts<OUT>(rc, p, rbc, lane);
  const bool quad_on = j < J;
  const int jc = quad_on ? j : J - 1;  // idle lanes repeat the last quad's loads
  v16i acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0;
  const uint4* bbase = xt + (size_t)(lane >> 5) * kMfmaTilePos + (lane & 31);
  const QuadInfo qs = LocateQuad(p, quad0 + (uint32_t)jc);
  const bool live = qs.valid > 0;
  auto do_chunk = [&](int chunk) {
    const int ks_first = kLoopK ? chunk * KC : 0;  // first k-step of the chunk; LDS row 0 is channel group 2 * ks_first
    // bit i of cmask: k-step ks_first + i holds a nonzero of this row block
    const uint32_t cmask = kLoopK ? (p.kmask[(size_t)rbc * p.kmask_words + (ks_first >> 5)] >> (ks_first & 31)) & ((1u << kLoopChunk) - 1u) : kmask;
    auto load_weights = [&](int i0, int i1) {
      // blocks of absent k-steps are never multiplied; their loads are clamped
#pragma unroll
      for (int i = i0; i < i1; ++i) {
        if (i < KC) {
          const int ksc = min(ks_first + i, p.ksteps - 1);
          a[i] = static_cast<const v4i*>(p.wblocks)[((size_t)rbc * p.ksteps + ksc) * 64 + lane];
        }
      }
    };
    // D[32 rows][32 cols] += A[32 x 32k] * B[32k x 32] for the chunk's k-steps [i0, i1)
    auto multiply = [&](int i0, int i1) {
      if (KSMAX != 32 && i1 - i0 == 4 && i1 <= KC && ((cmask >> i0) & 15u) == 15u) {
        // all four k-steps present: no branches, and the cells of the next
        // k-step are read from LDS while this one is multiplied (the
        // 32-k-step kernel has no registers left for the second set of cells)
        uint4 bq[2][4];
#pragma unroll
        for (int c = 0; c < 4; ++c) bq[0][c] = bbase[(size_t)(2 * i0) * kMfmaTilePos + c * 32];
#pragma unroll
        for (int i = i0; i < i1; ++i) {
          if (i + 1 < i1) {
#pragma unroll
            for (int c = 0; c < 4; ++c) bq[(i + 1 - i0) & 1][c] = bbase[(size_t)(2 * (i + 1)) * kMfmaTilePos + c * 32];
          }
          __builtin_amdgcn_sched_barrier(0);  // keeps the reads ahead of the multiplies
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const uint4 q = bq[(i - i0) & 1][c];
            acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i < KC ? i : 0], v4i{(int)q.x, (int)q.y, (int)q.z, (int)q.w}, acc[c], 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        return;
      }
#pragma unroll
      for (int i = i0; i < i1; ++i) {
        if (i < KC && (cmask & (1u << i))) {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const uint4 bq = bbase[(size_t)(2 * i) * kMfmaTilePos + c * 32];
            const v4i b = v4i{(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w};
            acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i < KC ? i : 0], b, acc[c], 0, 0, 0);
          }
        }
      }
    };
    // the previous chunk's tile is read until every wavefront has multiplied
    if (kLoopK && chunk > 0) __syncthreads();
    if (VEC) {
      // A pass of the workgroup stages 8 channel groups = 4 k-steps.  The
      // loads of up to four passes (activations, then that pass's weight
      // blocks) go out together; each pass is then committed to LDS and
      // multiplied as soon as its own loads have landed, while the later
      // ones are still in flight.
      constexpr int kPasses = (2 * KC + 7) / 8;
      constexpr int kBatch = kPasses < 4 ? kPasses : 4;
      uint32_t r[kBatch][16];
      // One straight-line instance per batch and addressing mode: loads
      // under per-pass conditions would be drained at every join.
      auto run_batch = [&](auto fast_c, int pass0) {
        constexpr bool kFast = decltype(fast_c)::value;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          LoadX<kFast>(r[u], p, qs, 2 * ks_first + 8 * (pass0 + u), kg0);
          load_weights(4 * (pass0 + u), 4 * (pass0 + u) + 4);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          CommitX<kFast>(r[u], xt, p, qs, kFast ? true : live, kFast ? (quad_on && live) : quad_on, 2 * ks_first + 8 * (pass0 + u), kg0, jc, 2 * ks_first);
          __syncthreads();
          if (wave_on) multiply(4 * (pass0 + u), 4 * (pass0 + u) + 4);
        }
      };
#pragma unroll
      for (int pass0 = 0; pass0 < kPasses; pass0 += kBatch) {
        if (pass0 > 0 && 2 * ks_first + 8 * pass0 >= 2 * p.ksteps) continue;
        if (p.small && 16 * (2 * ks_first + 8 * (pass0 + kBatch)) <= p.K) {
          run_batch(std::true_type(), pass0);
        } else {
          run_batch(std::false_type(), pass0);
        }
      }
    } else {
      load_weights(0, KC);
      StageMfmaBytes(xt, p, quad0 + (uint32_t)jc, quad_on, kg0, jc, 2 * ks_first, min(2 * (ks_first + KC), 2 * p.ksteps));
      __syncthreads();
      if (wave_on) multiply(0, KC);
    }
  };
  if (kLoopK) {
    const int n_chunks = (p.ksteps + KC - 1) / KC;
    for (int chunk = 0; chunk < n_chunks; ++chunk) do_chunk(chunk);
  } else {
    do_chunk(0);
  }
  if (!wave_on) return;
  if (!kEarlyConsts) LoadRowConsts<OUT>(rc, p, rbc, lane);
  MfmaFinish<OUT, ACT, VEC>(p, reinterpret_cast<uint32_t*>(xt + (size_t)2 * (kLoopK ? KC : p.ksteps) * kMfmaTilePos), acc, rc, rb, lane, quad0, J);
}

// Few input channels (at most 64, KSMAX <= 2): the channel groups of one
// tile fill only 2 * ksteps of the 8 group slots of a staging pass, so the
// workgroup takes T = 4 / ksteps neighbouring tiles at once (LDS: tile after
// tile) and each wavefront finishes T * RB / 4 (tile, row block) pairs with
// one set of weight blocks, RB = row blocks of the group (1, 2 or 4).
template <int KSMAX, int OUT, int ACT>
__device__ __forceinline__ void MfmaTilesFewChannels(const MfmaParams& p, uint4* xt, int wg_tile, int group, int wave) {
  const int tid = threadIdx.x, lane = tid & 63, j = tid & 31, kg0 = tid >> 5;
  const int T = p.sub_tiles;
  const int n_kg = 2 * p.ksteps;  // == 8 / T
  const int sub_l = kg0 / n_kg, kgl = kg0 - sub_l * n_kg;
  const int RB = min(4, p.row_blocks - 4 * group);
  const int rb = 4 * group + (wave & (RB - 1));
  const uint32_t kmask = p.kmask[(size_t)rb * p.kmask_words];
  RowConsts rc;
  LoadRowConsts<OUT>(rc, p, rb, lane);
  v4i a[KSMAX];
  const size_t tile_cells = (size_t)n_kg * kMfmaTilePos;
  {
    const QuadInfo qs = LocateQuad(p, ((uint32_t)wg_tile * T + sub_l) * 32u + j);
    const bool live = qs.valid > 0;
    uint32_t r[16];
    uint4* xs = xt + (size_t)sub_l * tile_cells;
    const bool fast = p.small && p.K == 32 * p.ksteps;
    if (fast) {
      LoadX<true>(r, p, qs, 0, kgl);
    } else {
      LoadX<false>(r, p, qs, 0, kgl);
    }
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) a[ks] = static_cast<const v4i*>(p.wblocks)[((size_t)rb * p.ksteps + min(ks, p.ksteps - 1)) * 64 + lane];
    if (fast) {
      CommitX<true>(r, xs, p, qs, true, live, 0, kgl, j);
    } else {
      CommitX<false>(r, xs, p, qs, live, true, 0, kgl, j);
    }
  }
  __syncthreads();
  uint32_t* stage = reinterpret_cast<uint32_t*>(xt + (size_t)T * tile_cells);
  for (int it = wave; it < T * RB; it += 4) {
    const int sub = it / RB;
    const uint32_t quad0 = ((uint32_t)wg_tile * T + sub) * 32u;
    if (quad0 >= p.total_quads) break;
    v16i acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[c][i] = 0;
    const uint4* bbase = xt + (size_t)sub * tile_cells + (size_t)(lane >> 5) * kMfmaTilePos + (lane & 31);
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
      if (kmask & (1u << ks)) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint4 bq = bbase[(size_t)(2 * ks) * kMfmaTilePos + c * 32];
          const v4i b = v4i{(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w};
          acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks], b, acc[c], 0, 0, 0);
        }
      }
    }
    MfmaFinish<OUT, ACT, true>(p, stage, acc, rc, rb, lane, quad0, 32);
  }
}

template <int KSMAX, int OUT, int ACT, bool VEC>
__device__ __forceinline__ void MfmaBody(const MfmaParams& p, uint4* xt) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Workgroups are handed to the 8 XCDs round robin.  Map the linear id so
  // that the workgroups sharing one activation tile (all row-block groups)
  // run on the same XCD one after the other: the tile is then fetched into
  // that XCD's L2 once.
  // Each XCD takes a contiguous range of tiles: cache lines that straddle
  // two neighbouring tiles are then fetched by one L2 instead of two.
  const int tile = XcdTile(p.tiles, p.row_groups);
  if (tile < 0) return;
  if (KSMAX <= 2 && VEC && p.sub_tiles > 1) {
    MfmaTilesFewChannels<(KSMAX <= 2 ? KSMAX : 1), OUT, (ACT < 0 ? 0 : ACT)>(p, xt, tile, (blockIdx.x >> 3) % p.row_groups, wave);
    return;
  }
  const int rb = ((blockIdx.x >> 3) % p.row_groups) * 4 + wave;
  const bool wave_on = rb < p.row_blocks;
  const int rbc = wave_on ? rb : p.row_blocks - 1;
  const uint32_t kmask = wave_on ? p.kmask[(size_t)rbc * p.kmask_words] : 0u;  // first 32 k-steps; chunked kernels read their own words
  MfmaTile<KSMAX, OUT, ACT, VEC>(p, xt, kmask, rb, rbc, wave_on, tile);
}

// ------------------------------------------------------ streaming block MFMA
// Large feature maps with 128 or 256 input channels (K = 32 * KSMAX, H*W a
// multiple of 16, whole row groups).  The grid is as large as the chip holds
// at once; a workgroup keeps one row group (its weight blocks stay in
// registers) and walks over tiles of its XCD's range.  While the epilogue of
// one tile runs (the vector-ALU bound part for int8 output) the activations
// of the workgroup's next tile are already on their way into registers:
//   barrier | loads(next) | epilogue + stores(current) | commit(next) | barrier | multiply(next)
// Loads, stores and the commit sit in one straight-line block, so the commit
// waits for exactly the loads (the stores issued after them may still be in
// flight).  Tiles are cut per image (the last tile of an image may hold fewer
// quads): every tile then takes the same path, and the lanes behind the last
// quad repeat it (same loads, same results, same store addresses).
struct StreamTile {
  uint32_t n;    // image
  uint32_t pp0;  // first position of the tile in its image
  int jv;        // quads of the tile that exist (a multiple of 4, at most 32)
};

__device__ __forceinline__ StreamTile LocateStreamTile(const MfmaParams& p, int t) {
  StreamTile s;
  s.n = (uint32_t)t / (uint32_t)p.stream_tpi;
  const uint32_t k = (uint32_t)t - s.n * (uint32_t)p.stream_tpi;
  s.pp0 = 128u * k;
  s.jv = min(32, p.qpi - 32 * (int)k);
  return s;
}

// acc = A (the wavefront's 32 rows) x B (the tile in LDS) over all k-steps.
template <int KSMAX>
__device__ __forceinline__ void StreamMultiply(v16i (&acc)[4], const v4i (&a)[KSMAX], const uint4* bbase, uint32_t kmask) {
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0;
  if (kmask == (1u << KSMAX) - 1u) {
    // every block present: no branches, the cells of the next k-step are
    // read while this one is multiplied
    uint4 bq[2][4];
#pragma unroll
    for (int c = 0; c < 4; ++c) bq[0][c] = bbase[c * 32];
#pragma unroll
    for (int i = 0; i < KSMAX; ++i) {
      if (i + 1 < KSMAX) {
#pragma unroll
        for (int c = 0; c < 4; ++c) bq[(i + 1) & 1][c] = bbase[(size_t)(2 * (i + 1)) * kMfmaTilePos + c * 32];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint4 q = bq[i & 1][c];
        acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], v4i{(int)q.x, (int)q.y, (int)q.z, (int)q.w}, acc[c], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < KSMAX; ++i) {
    if (kmask & (1u << i)) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint4 bq = bbase[(size_t)(2 * i) * kMfmaTilePos + c * 32];
        acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], v4i{(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w}, acc[c], 0, 0, 0);
      }
    }
  }
}

// Epilogue of one tile.  rcs: the row group's 128 scales followed by its 128
// biases in LDS; stage: the wavefront's 4 KB (int8 output only).
template <int OUT, int ACT>
__device__ __forceinline__ void StreamEpilogue(const MfmaParams& p, const v16i (&acc)[4], const float* rcs, uint32_t* stage, int wave, int rb, int lane, const StreamTile& s) {
  const int j = lane & 31, half = lane >> 5;
  const float* rs = rcs + wave * 32 + 4 * half;
  if (OUT == kOutI8) {
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const float4 sv = *reinterpret_cast<const float4*>(rs + 8 * g4);
      const float4 bv = *reinterpret_cast<const float4*>(rs + 128 + 8 * g4);
      const float sc[4] = {sv.x, sv.y, sv.z, sv.w}, bi[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for (int i = 0; i < 4; i += 2) {
        float f[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int c = 0; c < 4; ++c) f[h][c] = ActQuantF<ACT>(__builtin_fmaf((float)acc[c][4 * g4 + i + h], sc[i + h], bi[i + h]), p.act);
        uint32_t w0, w1;
        TruncPackI8x8(f[0][0], f[0][1], f[0][2], f[0][3], f[1][0], f[1][1], f[1][2], f[1][3], w0, w1);
        const int ro = 4 * half + 8 * g4 + i;  // row of the block; 32 dwords per row
        stage[ro * 32 + j] = w0;
        stage[(ro + 1) * 32 + j] = w1;
      }
    }
    // the same wavefront reads back: its LDS operations complete in order
    char* obase = static_cast<char*>(p.out) + (uint32_t)((s.n * (uint32_t)p.M + (uint32_t)rb * 32u) * (uint32_t)p.hw + s.pp0);
    const int chunk = min(lane & 7, (s.jv >> 2) - 1);  // 16 positions; chunks behind the tile's end repeat its last one
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 8 * i + (lane >> 3);
      const uint4 v = *reinterpret_cast<const uint4*>(stage + row * 32 + chunk * 4);
      StreamStore(make_int4((int)v.x, (int)v.y, (int)v.z, (int)v.w), obase + (uint32_t)row * (uint32_t)p.hw + chunk * 16);
    }
  } else {
    const int jc = min(j, s.jv - 1);
    char* lane_base = static_cast<char*>(p.out) + (uint32_t)(((s.n * (uint32_t)p.M + (uint32_t)rb * 32u + 4u * half) * (uint32_t)p.hw + s.pp0 + 4u * jc) * 4u);
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const float4 sv = *reinterpret_cast<const float4*>(rs + 8 * g4);
      const float4 bv = *reinterpret_cast<const float4*>(rs + 128 + 8 * g4);
      const float sc[4] = {sv.x, sv.y, sv.z, sv.w}, bi[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = ActivateT<ACT>(__builtin_fmaf((float)acc[c][4 * g4 + i], sc[i], bi[i]), p.act);
        StreamStore(make_float4(v[0], v[1], v[2], v[3]), lane_base + (size_t)(8 * g4 + i) * (size_t)p.hw * 4u);
      }
    }
  }
}

template <int KSMAX, int OUT, int ACT>
__device__ __forceinline__ void StreamBody(const MfmaParams& p, uint4* xt) {
  const int tid = threadIdx.x, lane = tid & 63, j = tid & 31, kg0 = tid >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int group = slot % p.row_groups, tl = slot / p.row_groups;
  const int lo = (int)(((int64_t)xcd * p.stream_tiles) >> 3), hi = (int)(((int64_t)(xcd + 1) * p.stream_tiles) >> 3);
  int t = lo + tl;
  if (t >= hi) return;
  const int rb = group * 4 + wave;
  const uint32_t kmask = p.kmask[(size_t)rb * p.kmask_words] & ((1u << KSMAX) - 1u);
  v4i a[KSMAX];
#pragma unroll
  for (int ks = 0; ks < KSMAX; ++ks) a[ks] = static_cast<const v4i*>(p.wblocks)[((size_t)rb * p.ksteps + ks) * 64 + lane];
  // LDS: activation tile | the row group's scales and biases | int8 staging
  float* rcs = reinterpret_cast<float*>(xt + (size_t)2 * KSMAX * kMfmaTilePos);
  uint32_t* stage = reinterpret_cast<uint32_t*>(rcs + 256) + wave * 1024;
  if (tid < 128) {
    rcs[tid] = p.scale[group * 128 + tid];
    rcs[128 + tid] = p.bias[group * 128 + tid];
  }
  constexpr int kPasses = KSMAX / 4;
  uint32_t r[kPasses][16];
  const QuadInfo none = {0u, 0u, 4};
  auto issue = [&](const StreamTile& s) {
    const QuadInfo q = {s.n, s.pp0 + 4u * (uint32_t)min(j, s.jv - 1), 4};
#pragma unroll
    for (int u = 0; u < kPasses; ++u) LoadX<true>(r[u], p, q, 8 * u, kg0);
  };
  auto commit = [&]() {
#pragma unroll
    for (int u = 0; u < kPasses; ++u) CommitX<true>(r[u], xt, p, none, true, true, 8 * u, kg0, j);
  };
  const uint4* bbase = xt + (size_t)(lane >> 5) * kMfmaTilePos + (lane & 31);
  v16i acc[4];
  StreamTile cur = LocateStreamTile(p, t);
  issue(cur);
  commit();
  __syncthreads();
  StreamMultiply<KSMAX>(acc, a, bbase, kmask);
  for (t += p.stream_lanes; t < hi; t += p.stream_lanes) {
    const StreamTile next = LocateStreamTile(p, t);
    __syncthreads();  // every wavefront has read the current tile
    issue(next);
    __builtin_amdgcn_sched_barrier(0);  // the loads stay ahead of the epilogue
    StreamEpilogue<OUT, ACT>(p, acc, rcs, stage, wave, rb, lane, cur);
    __builtin_amdgcn_sched_barrier(0);
    commit();
    __syncthreads();
    StreamMultiply<KSMAX>(acc, a, bbase, kmask);
    cur = next;
  }
  StreamEpilogue<OUT, ACT>(p, acc, rcs, stage, wave, rb, lane, cur);
}

template <int KSMAX, int OUT>
__global__ void __launch_bounds__(256, (KSMAX == 4 ? 3 : 2)) StreamMfmaKernel(const MfmaParams p) {
  extern __shared__ uint4 xt[];
  DispatchAct(p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    StreamBody<KSMAX, OUT, ACT>(p, xt);
  });
}

// At least two workgroups per CU (two wavefronts per SIMD): caps the kernel
// at 256 VGPRs.
template <int KSMAX, int OUT>
__global__ void __launch_bounds__(256, (KSMAX == 4 ? 4 : 2)) BlockMfmaKernel(const MfmaParams p) {
  extern __shared__ uint4 xt[];
  if (!p.vec) {
    MfmaBody<KSMAX, OUT, -1, false>(p, xt);
    return;
  }
  DispatchAct(OUT == kOutAcc32 ? 0 : p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    MfmaBody<KSMAX, OUT, ACT, true>(p, xt);
  });
}

#endif  // PL_PART_MFMA_ANY

// ------------------------------------------------------------- launch glue
// LaunchWithLds (launch_lds.h) enables dynamic LDS above the default limit per
// kernel function and device.

#if PL_PART_WALK
template <bool INT8, int OUT, int NR>
hipError_t WalkByTile(const WalkConfig& cfg, const WalkParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  switch (cfg.tile_pos) {
    case 16:
      return LaunchWithLds(RowWalkKernel<INT8, OUT, NR, 16>, grid, block, lds, s, p);
    case 32:
      return LaunchWithLds(RowWalkKernel<INT8, OUT, NR, 32>, grid, block, lds, s, p);
    case 64:
      return LaunchWithLds(RowWalkKernel<INT8, OUT, NR, 64>, grid, block, lds, s, p);
    case 128:
      return LaunchWithLds(RowWalkKernel<INT8, OUT, NR, 128>, grid, block, lds, s, p);
    case 256:
      return LaunchWithLds(RowWalkKernel<INT8, OUT, NR, 256>, grid, block, lds, s, p);
    default:
      return hipErrorInvalidValue;
  }
}

template <bool INT8, int OUT>
hipError_t WalkByRows(const WalkConfig& cfg, const WalkParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  return cfg.nrows == 2 ? WalkByTile<INT8, OUT, 2>(cfg, p, grid, block, lds, s)
                        : WalkByTile<INT8, OUT, 1>(cfg, p, grid, block, lds, s);
}
#endif  // PL_PART_WALK

#if PL_PART_MFMA_ANY
template <int OUT>
hipError_t MfmaByKs(int ks_max, const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  switch (ks_max) {
    case 2:
      return LaunchWithLds(BlockMfmaKernel<2, OUT>, grid, block, lds, s, p);
    case 4:
      return LaunchWithLds(BlockMfmaKernel<4, OUT>, grid, block, lds, s, p);
    case 8:
      return LaunchWithLds(BlockMfmaKernel<8, OUT>, grid, block, lds, s, p);
    case 16:
      return LaunchWithLds(BlockMfmaKernel<16, OUT>, grid, block, lds, s, p);
    case 32:
      return LaunchWithLds(BlockMfmaKernel<32, OUT>, grid, block, lds, s, p);
    case 64:
      return LaunchWithLds(BlockMfmaKernel<64, OUT>, grid, block, lds, s, p);
    default:
      return hipErrorInvalidValue;
  }
}
template <int OUT>
hipError_t StreamByKs(const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  if (p.ksteps == 4) return LaunchWithLds(StreamMfmaKernel<4, OUT>, grid, block, lds, s, p);
  if (p.ksteps == 8) return LaunchWithLds(StreamMfmaKernel<8, OUT>, grid, block, lds, s, p);
  return hipErrorInvalidValue;
}
#endif  // PL_PART_MFMA_ANY

}  // namespace

// The block MFMA kernels of each output kind are compiled in their own
// translation unit (see the part macros at the top of this file).
hipError_t LaunchMfmaF32(int ks_max, const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s);
hipError_t LaunchMfmaI8(int ks_max, const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s);
hipError_t LaunchMfmaAcc32(int ks_max, const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s);
hipError_t LaunchStreamF32(const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s);
hipError_t LaunchStreamI8(const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s);

#if PL_PART_MFMA_F32
hipError_t LaunchMfmaF32(int ks_max, const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) { return MfmaByKs<kOutF32>(ks_max, p, grid, block, lds, s); }
hipError_t LaunchStreamF32(const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) { return StreamByKs<kOutF32>(p, grid, block, lds, s); }
#endif
#if PL_PART_MFMA_I8
hipError_t LaunchMfmaI8(int ks_max, const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) { return MfmaByKs<kOutI8>(ks_max, p, grid, block, lds, s); }
hipError_t LaunchStreamI8(const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) { return StreamByKs<kOutI8>(p, grid, block, lds, s); }
#endif
#if PL_PART_MFMA_ACC32
hipError_t LaunchMfmaAcc32(int ks_max, const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) { return MfmaByKs<kOutAcc32>(ks_max, p, grid, block, lds, s); }
#endif

#if PL_PART_WALK
hipError_t LaunchRowWalk(const WalkConfig& cfg, const WalkParams& p, hipStream_t stream) {
  if (p.P == 0 || p.n_groups == 0) return hipSuccess;
  const size_t lds = (size_t)(p.kd + (cfg.int8 ? 0 : 1)) * cfg.tile_pos * 4;
  if (lds > (size_t)kMaxLdsBytes) return hipErrorInvalidValue;
  if (cfg.threads % cfg.tile_pos != 0 && cfg.tile_pos % cfg.threads != 0) return hipErrorInvalidValue;
  if (cfg.threads < cfg.tile_pos) return hipErrorInvalidValue;
  const uint32_t tiles = (p.P + cfg.tile_pos - 1) / cfg.tile_pos;
  WalkParams q = p;
  q.tiles = (int)tiles;
  q.slices = cfg.slices;
  dim3 grid(8u * (uint32_t)cfg.slices * ((tiles + 7) / 8)), block(cfg.threads);
  if (!cfg.int8) {
    if (cfg.out_kind != kOutF32) return hipErrorInvalidValue;
    return WalkByRows<false, kOutF32>(cfg, q, grid, block, lds, stream);
  }
  switch (cfg.out_kind) {
    case kOutF32:
      return WalkByRows<true, kOutF32>(cfg, q, grid, block, lds, stream);
    case kOutI8:
      return WalkByRows<true, kOutI8>(cfg, q, grid, block, lds, stream);
    case kOutAcc32:
      return WalkByRows<true, kOutAcc32>(cfg, q, grid, block, lds, stream);
    default:
      return hipErrorInvalidValue;
  }
}

hipError_t LaunchBlockMfma(const MfmaConfig& cfg, const MfmaParams& p, hipStream_t stream) {
  if (p.P == 0 || p.row_blocks == 0) return hipSuccess;
  if (p.ksteps > cfg.ks_max && cfg.ks_max <= 32) return hipErrorInvalidValue;  // ks_max 64 = any count, kLoopChunk at a time
  if (cfg.tile_quads < 1 || cfg.tile_quads > 32 || p.hw < 1) return hipErrorInvalidValue;
  MfmaParams q = p;
  q.qpi = (p.hw + 3) / 4;
  q.total_quads = (p.P / (uint32_t)p.hw) * (uint32_t)q.qpi;
  q.vec = p.hw >= 4;
  q.quad_aligned = p.hw % 4 == 0;
  q.tile_quads = cfg.tile_quads;
  uint32_t tiles = (q.total_quads + cfg.tile_quads - 1) / cfg.tile_quads;
  q.row_groups = (p.row_blocks + 3) / 4;
  // Streaming variant: large maps with 128 or 256 channels, whole row groups,
  // 16-byte row pieces, tiles cut per image with at most 15 % of the quads of
  // the per-image tiling empty (28 x 28 maps: 12.5 %), and at least one tile
  // for every resident workgroup.
  if (cfg.stream && (cfg.out_kind == kOutI8 || cfg.out_kind == kOutF32) && (p.ksteps == 4 || p.ksteps == 8) && p.K == 32 * p.ksteps && cfg.ks_max == p.ksteps &&
      p.hw % 16 == 0 && p.small && p.row_blocks % 4 == 0 && p.M == 32 * p.row_blocks && cfg.tile_quads == 32 && reinterpret_cast<uintptr_t>(p.out) % 16 == 0) {
    const int tpi = (q.qpi + 31) / 32;
    const int64_t stream_tiles = (int64_t)(p.P / (uint32_t)p.hw) * tpi;
    const int per_cu = p.ksteps == 4 ? 3 : 2;  // resident workgroups per CU, by registers
    int lanes = std::max(1, cfg.cus * per_cu / 8 / q.row_groups);
    if (stream_tiles < (1ll << 30) && (cfg.stream == 2 || (tpi * 32 * 100 <= q.qpi * 115 && stream_tiles >= (int64_t)8 * lanes))) {
      lanes = (int)std::min<int64_t>(lanes, (stream_tiles + 7) / 8);
      q.stream_tpi = tpi;
      q.stream_tiles = (int)stream_tiles;
      q.stream_lanes = lanes;
      size_t slds = (size_t)2 * p.ksteps * kMfmaTilePos * 16 + 1024 + (cfg.out_kind == kOutI8 ? 16384 : 0);
      dim3 sgrid(8u * (uint32_t)q.row_groups * (uint32_t)lanes), sblock(256);
      return cfg.out_kind == kOutI8 ? LaunchStreamI8(q, sgrid, sblock, slds, stream) : LaunchStreamF32(q, sgrid, sblock, slds, stream);
    }
  }
  // at most 64 input channels: a workgroup takes 4 / ksteps tiles at once
  // (every row group must have 1, 2 or 4 row blocks, and enough workgroups
  // must remain to fill the chip)
  q.sub_tiles = 1;
  if (cfg.ks_max == 2 && cfg.sub_tiles && q.vec && cfg.tile_quads == 32 && (p.row_blocks % 4 == 0 || p.row_blocks <= 2)) {
    const uint32_t t = 4u / (uint32_t)p.ksteps;
    if (cfg.sub_tiles == 2 || (tiles / t) * q.row_groups >= 1024u) q.sub_tiles = (int)t;
  }
  tiles = (tiles + q.sub_tiles - 1) / q.sub_tiles;
  q.tiles = (int)tiles;  // workgroup-level tiles
  size_t lds = (size_t)q.sub_tiles * 2 * (cfg.ks_max > 32 ? kLoopChunk : p.ksteps) * kMfmaTilePos * 16;
  if (lds > (size_t)kMaxLdsBytes) return hipErrorInvalidValue;
  // int8 output: 4 KB per wavefront behind the activation tile to widen stores
  q.i8_stage = cfg.out_kind == kOutI8 && cfg.i8_wide_stores && lds + 16384 <= (size_t)kMaxLdsBytes;
  if (q.i8_stage) lds += 16384;
  dim3 grid(8u * q.row_groups * ((tiles + 7) / 8)), block(256);  // one workgroup per (tile, row group)
  switch (cfg.out_kind) {
    case kOutF32:
      return LaunchMfmaF32(cfg.ks_max, q, grid, block, lds, stream);
    case kOutI8:
      return LaunchMfmaI8(cfg.ks_max, q, grid, block, lds, stream);
    case kOutAcc32:
      return LaunchMfmaAcc32(cfg.ks_max, q, grid, block, lds, stream);
    default:
      return hipErrorInvalidValue;
  }
}
#endif  // PL_PART_WALK

}  // namespace pl
