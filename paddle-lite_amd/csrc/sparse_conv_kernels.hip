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
#include "sparse_conv_kernels.h"

#include <atomic>
#include <type_traits>

// Phase marks for tuning builds; compiled out of the library.
#ifndef PL_PHASE_MARK
#define PL_PHASE_MARK(i)
#endif

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

// ---------------------------------------------------------------- epilogue
__device__ __forceinline__ float Activate(float v, const DevAct& a) {
  switch (a.type) {
    case 1:
      return fmaxf(v, 0.0f);
    case 2:
      return fminf(fmaxf(v, 0.0f), a.relu6_coef);
    case 4:
      return (v >= 0.0f) ? v : v * a.leaky_alpha;
    case 10: {
      float gate = fminf(fmaxf(v + a.hs_offset, 0.0f), a.hs_threshold);
      return (v * a.hs_inv_scale) * gate;
    }
    default:
      return v;
  }
}

// Same, with the activation fixed at compile time; DispatchAct turns the
// run-time type into that constant once per kernel instead of once per value.
template <int ACT>
__device__ __forceinline__ float ActivateT(float v, const DevAct& a) {
  if (ACT == 1) return fmaxf(v, 0.0f);
  if (ACT == 2) return fminf(fmaxf(v, 0.0f), a.relu6_coef);
  if (ACT == 4) return (v >= 0.0f) ? v : v * a.leaky_alpha;
  if (ACT == 10) {
    float gate = fminf(fmaxf(v + a.hs_offset, 0.0f), a.hs_threshold);
    return (v * a.hs_inv_scale) * gate;
  }
  return v;
}

template <typename F>
__device__ __forceinline__ void DispatchAct(int type, F&& f) {
  switch (type) {
    case 1:
      f(std::integral_constant<int, 1>());
      break;
    case 2:
      f(std::integral_constant<int, 2>());
      break;
    case 4:
      f(std::integral_constant<int, 4>());
      break;
    case 10:
      f(std::integral_constant<int, 10>());
      break;
    default:
      f(std::integral_constant<int, 0>());
      break;
  }
}

__device__ __forceinline__ int QuantizeI8(float v) {
  v = fmaxf(v, -127.0f);
  float r = roundf(v);  // half away from zero
  r = fminf(r, 127.0f);
  return static_cast<int>(r);
}

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
// fp32: tile[k][TP] floats.  int8: tile[q][TP] dwords, dword = channels
// 4q..4q+3 of one position (channels past K read as zero).
template <bool INT8, int TP>
__device__ __forceinline__ void StageTile(uint32_t* tile, const WalkParams& p, uint32_t tile0) {
  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  if (p.vec) {
    constexpr int TPV = TP / 4;  // groups of four positions per row
    const int j4 = tid % TPV;
    const uint32_t g = tile0 + 4u * j4;
    const bool live = g < p.P;
    const uint32_t n = live ? g / (uint32_t)p.hw : 0u;
    const uint32_t pp = live ? g % (uint32_t)p.hw : 0u;
    for (int k = tid / TPV; k < p.kd; k += nthreads / TPV) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (live) {
        if (!INT8) {
          const float* src = static_cast<const float*>(p.x) + ((size_t)n * p.K + k) * p.hw + pp;
          v = *reinterpret_cast<const uint4*>(src);
        } else {
          const int8_t* src = static_cast<const int8_t*>(p.x) + ((size_t)n * p.K + 4 * k) * p.hw + pp;
          uint32_t r0 = *reinterpret_cast<const uint32_t*>(src);
          uint32_t r1 = (4 * k + 1 < p.K) ? *reinterpret_cast<const uint32_t*>(src + p.hw) : 0u;
          uint32_t r2 = (4 * k + 2 < p.K) ? *reinterpret_cast<const uint32_t*>(src + 2 * (size_t)p.hw) : 0u;
          uint32_t r3 = (4 * k + 3 < p.K) ? *reinterpret_cast<const uint32_t*>(src + 3 * (size_t)p.hw) : 0u;
          Transpose4x4(r0, r1, r2, r3);
          v = make_uint4(r0, r1, r2, r3);
        }
      }
      *reinterpret_cast<uint4*>(tile + (size_t)k * TP + 4 * j4) = v;
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
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
      } else if (PPL == 2) {
        *reinterpret_cast<float2*>(dst) = make_float2(v[0], v[1]);
      } else {
        dst[0] = v[0];
      }
    } else if (OUT == kOutI8) {
      int8_t* dst = static_cast<int8_t*>(p.out) + idx;
      if (PPL == 4) {
        uint32_t w = (uint32_t)(QuantizeI8(v[0]) & 0xff) | ((uint32_t)(QuantizeI8(v[1]) & 0xff) << 8) |
                     ((uint32_t)(QuantizeI8(v[2]) & 0xff) << 16) | ((uint32_t)(QuantizeI8(v[3]) & 0xff) << 24);
        *reinterpret_cast<uint32_t*>(dst) = w;
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
template <bool INT8, int OUT, int NR, int TP>
__global__ void __launch_bounds__(1024) RowWalkKernel(const WalkParams p) {
  extern __shared__ uint32_t tile[];
  constexpr int PPL = TP >= 64 ? TP / 64 : 1;  // positions per lane
  const uint32_t tile0 = blockIdx.x * (uint32_t)TP;

  StageTile<INT8, TP>(tile, p, tile0);
  __syncthreads();

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nwaves = blockDim.x >> 6;
  const int g_begin = blockIdx.y * p.groups_per_slice;
  const int g_end = min(p.n_groups, g_begin + p.groups_per_slice);
  const bool lane_on = (TP >= 64) || (lane < TP);
  const uint32_t* xbase = tile + (lane_on ? lane * PPL : 0);

  for (int g = g_begin + wave; g < g_end; g += nwaves) {
    const DevGroup grp = p.groups[g];
    const uint32_t* __restrict__ kp = p.kidx + grp.first;
    const uint32_t* __restrict__ wp = p.wts + (size_t)grp.first * NR;

    float f0[PPL], f1[PPL];
    int a0[PPL], a1[PPL];
#pragma unroll
    for (int j = 0; j < PPL; ++j) {
      a0[j] = a1[j] = 0;
      f0[j] = f1[j] = 0.0f;
    }
    if (!INT8) {
      const float b0 = p.bias ? p.bias[grp.row0] : 0.0f;
      const float b1 = (p.bias && NR == 2 && grp.nrows == 2) ? p.bias[grp.row0 + 1] : 0.0f;
#pragma unroll
      for (int j = 0; j < PPL; ++j) {
        f0[j] = b0;
        f1[j] = b1;
      }
    }

#pragma unroll 4
    for (uint32_t e = 0; e < grp.count; ++e) {
      const uint32_t k = kp[e];
      const uint32_t w0 = wp[(size_t)e * NR];
      const uint32_t w1 = (NR == 2) ? wp[(size_t)e * NR + 1] : 0u;
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
          const float s = p.scale[row];
          const float b = p.bias ? p.bias[row] : 0.0f;
#pragma unroll
          for (int j = 0; j < PPL; ++j) v[j] = Activate(__builtin_fmaf((float)acc[j], s, b), p.act);
        }
      } else {
        const float* f = r == 0 ? f0 : f1;
#pragma unroll
        for (int j = 0; j < PPL; ++j) v[j] = Activate(f[j], p.act);
      }
      StoreRow<OUT, PPL>(p, row, gpos, v, acc);
    }
  }
}

// -------------------------------------------------------------- block MFMA
// LDS layout: xt[kg][slot] 16-byte cells, kg = group of 16 input channels,
// slot = c*32 + j holds position 4*j + c of the 128-position tile, so that
// MFMA column j of the four accumulators c = 0..3 are four consecutive
// positions of one output row (one 16-byte fp32 store, one dword int8 store).

// Stage with aligned dword loads (hw % 4 == 0).  Every load is unconditional
// so that all loads of a batch are in flight together.  FAST: all channel
// groups of the batch are complete, the tile lies inside the tensor and the
// tensor is below 2 GB, so an address is a uniform base plus one 32-bit
// per-lane offset (no per-load address arithmetic on the vector ALU).
// Otherwise addresses are clamped and the results masked.
template <int UNITS, bool FAST>
__device__ __forceinline__ void StageMfmaVec(uint4* xt, const MfmaParams& p, uint32_t tile0, int kg_base, int kg_lane, int j) {
  const int n_kg = 2 * p.ksteps;
  const uint32_t g = tile0 + 4u * j;
  const bool live = FAST || g < p.P;
  const uint32_t gs = live ? g : 0u;
  const uint32_t n = gs / (uint32_t)p.hw, pp = gs % (uint32_t)p.hw;
  uint32_t r[UNITS][16];
  if (FAST) {
    const uint32_t voff = (n * (uint32_t)p.K + 16u * (uint32_t)kg_lane) * (uint32_t)p.hw + pp;
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int8_t* sbase = p.x + (size_t)(16 * (kg_base + 8 * u) + i) * (size_t)p.hw;  // uniform
        r[u][i] = *reinterpret_cast<const uint32_t*>(sbase + voff);
      }
    }
  } else {
    const int8_t* col = p.x + (size_t)n * p.K * p.hw + pp;
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
      const int kg = kg_base + kg_lane + 8 * u;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int ch = min(16 * kg + i, p.K - 1);
        r[u][i] = *reinterpret_cast<const uint32_t*>(col + (size_t)ch * p.hw);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    const int kg = kg_base + kg_lane + 8 * u;
    if (!FAST) {
#pragma unroll
      for (int i = 0; i < 16; ++i) r[u][i] = (live && 16 * kg + i < p.K) ? r[u][i] : 0u;
    }
#pragma unroll
    for (int b = 0; b < 4; ++b) Transpose4x4(r[u][4 * b], r[u][4 * b + 1], r[u][4 * b + 2], r[u][4 * b + 3]);
    // now r[u][4b + c] = channels 16kg+4b..+3 of position 4j+c
    if (FAST || kg < n_kg) {
#pragma unroll
      for (int c = 0; c < 4; ++c) xt[(size_t)kg * kMfmaTilePos + c * 32 + j] = make_uint4(r[u][c], r[u][4 + c], r[u][8 + c], r[u][12 + c]);
    }
  }
}

// Any hw: byte loads.
__device__ __forceinline__ void StageMfmaBytes(uint4* xt, const MfmaParams& p, uint32_t tile0, int kg0, int kg_step, int j) {
  const int n_kg = 2 * p.ksteps;
  const uint32_t g = tile0 + 4u * j;
  for (int kg = kg0; kg < n_kg; kg += kg_step) {
    for (int c = 0; c < 4; ++c) {
      const uint32_t gc = g + c;
      uint32_t d[4] = {0, 0, 0, 0};
      if (gc < p.P) {
        const uint32_t n = gc / (uint32_t)p.hw, pp = gc % (uint32_t)p.hw;
        const int8_t* col = p.x + (size_t)n * p.K * p.hw + pp;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int ch = 16 * kg + i;
          const uint32_t b = (ch < p.K) ? (uint32_t)(uint8_t)col[(size_t)ch * p.hw] : 0u;
          d[i >> 2] |= b << (8 * (i & 3));
        }
      }
      xt[(size_t)kg * kMfmaTilePos + c * 32 + j] = make_uint4(d[0], d[1], d[2], d[3]);
    }
  }
}

// Accumulator register r of lane l is output row 8*(r/4) + 4*(l/32) + r%4 of
// the 32-row block, column l%32; the four accumulators are four consecutive
// positions.
template <int OUT, int ACT, bool VEC>
__device__ __forceinline__ void MfmaEpilogue(const MfmaParams& p, const v16i (&acc)[4], int rb, int lane, uint32_t tile0) {
  const uint32_t g = tile0 + 4u * (lane & 31);
  if (g >= p.P) return;
  const uint32_t n = g / (uint32_t)p.hw, pp = g % (uint32_t)p.hw;
  const int row_base = rb * 32 + 4 * (lane >> 5);
  if (VEC && p.small && rb * 32 + 32 <= p.M) {
    // all 32 rows exist and byte offsets fit 32 bits: uniform row base plus
    // one per-lane offset
    constexpr uint32_t kElem = OUT == kOutI8 ? 1u : 4u;
    const uint32_t voff = ((n * (uint32_t)p.M + (uint32_t)row_base) * (uint32_t)p.hw + pp) * kElem;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int ro = 8 * (r >> 2) + (r & 3);
      char* dst = static_cast<char*>(p.out) + (size_t)ro * (size_t)p.hw * kElem + voff;
      int q[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) q[c] = acc[c][r];
      if (OUT == kOutAcc32) {
        StreamStore(make_int4(q[0], q[1], q[2], q[3]), dst);
      } else {
        const float s = p.scale[row_base + ro], b = p.bias[row_base + ro];
        float v[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = ActivateT<ACT>(__builtin_fmaf((float)q[c], s, b), p.act);
        if (OUT == kOutF32) {
          StreamStore(make_float4(v[0], v[1], v[2], v[3]), dst);
        } else {
          uint32_t w = (uint32_t)(QuantizeI8(v[0]) & 0xff) | ((uint32_t)(QuantizeI8(v[1]) & 0xff) << 8) |
                       ((uint32_t)(QuantizeI8(v[2]) & 0xff) << 16) | ((uint32_t)(QuantizeI8(v[3]) & 0xff) << 24);
          StreamStore(w, dst);
        }
      }
    }
    return;
  }
  float sc[16], bi[16];
  if (OUT != kOutAcc32) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = row_base + 8 * (r >> 2) + (r & 3);  // scale / bias are padded to 32 rows per block
      sc[r] = p.scale[row];
      bi[r] = p.bias[row];
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = row_base + 8 * (r >> 2) + (r & 3);
    if (row >= p.M) continue;
    float v[4];
    int q[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) q[c] = acc[c][r];
    if (OUT != kOutAcc32) {
#pragma unroll
      for (int c = 0; c < 4; ++c) v[c] = ActivateT<ACT>(__builtin_fmaf((float)q[c], sc[r], bi[r]), p.act);
    }
    if (VEC) {
      const size_t idx = ((size_t)n * p.M + row) * p.hw + pp;
      if (OUT == kOutF32) {
        *reinterpret_cast<float4*>(static_cast<float*>(p.out) + idx) = make_float4(v[0], v[1], v[2], v[3]);
      } else if (OUT == kOutI8) {
        uint32_t w = (uint32_t)(QuantizeI8(v[0]) & 0xff) | ((uint32_t)(QuantizeI8(v[1]) & 0xff) << 8) |
                     ((uint32_t)(QuantizeI8(v[2]) & 0xff) << 16) | ((uint32_t)(QuantizeI8(v[3]) & 0xff) << 24);
        *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(p.out) + idx) = w;
      } else {
        *reinterpret_cast<int4*>(static_cast<int*>(p.out) + idx) = make_int4(q[0], q[1], q[2], q[3]);
      }
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint32_t gc = g + c;
        if (gc < p.P) {
          const uint32_t nc = gc / (uint32_t)p.hw, pc = gc % (uint32_t)p.hw;
          StoreOne<OUT>(p.out, ((size_t)nc * p.M + row) * p.hw + pc, v[c], q[c]);
        }
      }
    }
  }
}

template <int KSMAX, int OUT>
__global__ void __launch_bounds__(256) BlockMfmaKernel(const MfmaParams p) {
  extern __shared__ uint4 xt[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Workgroups are handed to the 8 XCDs round robin.  Map the linear id so
  // that the workgroups sharing one activation tile (all row-block groups)
  // run on the same XCD one after the other: the tile is then fetched into
  // that XCD's L2 once.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int tile = (slot / p.row_groups) * 8 + xcd;
  if (tile >= p.tiles) return;
  const uint32_t tile0 = (uint32_t)tile * (uint32_t)kMfmaTilePos;
  const int rb = (slot % p.row_groups) * 4 + wave;
  const bool wave_on = rb < p.row_blocks;
  const int rbc = wave_on ? rb : p.row_blocks - 1;
  PL_PHASE_MARK(0);

  // weight blocks of this wavefront's 32 rows -> registers (blocks of absent
  // k-steps are never multiplied; their loads are clamped to a valid block)
  const uint32_t kmask = wave_on ? p.kmask[rbc] : 0u;
  v4i a[KSMAX];
#pragma unroll
  for (int ks = 0; ks < KSMAX; ++ks) {
    const int ksc = min(ks, p.ksteps - 1);
    a[ks] = static_cast<const v4i*>(p.wblocks)[((size_t)rbc * p.ksteps + ksc) * 64 + lane];
  }

  PL_PHASE_MARK(1);
  // ---- stage 128 positions x (32*ksteps) channels, channel-innermost
  {
    const int j = tid & 31;    // position quad of the tile
    const int kg0 = tid >> 5;  // 8 channel groups per pass of the workgroup
    if (p.vec) {
      constexpr int kPasses = (2 * KSMAX + 7) / 8;  // passes that cover 2*KSMAX groups
      constexpr int kBatch = kPasses < 4 ? kPasses : 4;
      const bool inside = p.small && tile0 + (uint32_t)kMfmaTilePos <= p.P;
#pragma unroll
      for (int pass = 0; pass < kPasses; pass += kBatch) {
        if (8 * pass < 2 * p.ksteps) {
          if (inside && 16 * 8 * (pass + kBatch) <= p.K) {
            StageMfmaVec<kBatch, true>(xt, p, tile0, 8 * pass, kg0, j);
          } else {
            StageMfmaVec<kBatch, false>(xt, p, tile0, 8 * pass, kg0, j);
          }
        }
      }
    } else {
      StageMfmaBytes(xt, p, tile0, kg0, 8, j);
    }
  }
  PL_PHASE_MARK(2);
  __syncthreads();
  PL_PHASE_MARK(3);
  if (!wave_on) return;

  // ---- multiply: D[32 rows][32 cols] += A[32 x 32k] * B[32k x 32], four
  //      column blocks
  v16i acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0;

  const uint4* bbase = xt + (size_t)(lane >> 5) * kMfmaTilePos + (lane & 31);
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

  PL_PHASE_MARK(4);
  DispatchAct(OUT == kOutAcc32 ? 0 : p.act.type, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
    if (p.vec) {
      MfmaEpilogue<OUT, ACT, true>(p, acc, rb, lane, tile0);
    } else {
      MfmaEpilogue<OUT, ACT, false>(p, acc, rb, lane, tile0);
    }
  });
  PL_PHASE_MARK(5);
}

// ------------------------------------------------------------- launch glue
// Dynamic LDS above the default limit has to be enabled per kernel and
// device; remember what was already enabled (one static per instantiation).
template <typename Kernel, typename Params>
hipError_t LaunchWithLds(Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const Params& p) {
  if (lds > 48 * 1024) {
    constexpr int kMaxDevices = 64;
    static std::atomic<size_t> enabled[kMaxDevices];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices || enabled[dev].load(std::memory_order_acquire) < lds) {
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return e;
      if (dev >= 0 && dev < kMaxDevices) enabled[dev].store(lds, std::memory_order_release);
    }
  }
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
  return hipGetLastError();
}

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

template <int OUT>
hipError_t MfmaByKs(const MfmaConfig& cfg, const MfmaParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  switch (cfg.ks_max) {
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
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace

hipError_t LaunchRowWalk(const WalkConfig& cfg, const WalkParams& p, hipStream_t stream) {
  if (p.P == 0 || p.n_groups == 0) return hipSuccess;
  const size_t lds = (size_t)p.kd * cfg.tile_pos * 4;
  if (lds > (size_t)kMaxLdsBytes) return hipErrorInvalidValue;
  if (cfg.threads % cfg.tile_pos != 0 && cfg.tile_pos % cfg.threads != 0) return hipErrorInvalidValue;
  if (cfg.threads < cfg.tile_pos) return hipErrorInvalidValue;
  const uint32_t tiles = (p.P + cfg.tile_pos - 1) / cfg.tile_pos;
  dim3 grid(tiles, cfg.slices), block(cfg.threads);
  if (!cfg.int8) {
    if (cfg.out_kind != kOutF32) return hipErrorInvalidValue;
    return WalkByRows<false, kOutF32>(cfg, p, grid, block, lds, stream);
  }
  switch (cfg.out_kind) {
    case kOutF32:
      return WalkByRows<true, kOutF32>(cfg, p, grid, block, lds, stream);
    case kOutI8:
      return WalkByRows<true, kOutI8>(cfg, p, grid, block, lds, stream);
    case kOutAcc32:
      return WalkByRows<true, kOutAcc32>(cfg, p, grid, block, lds, stream);
    default:
      return hipErrorInvalidValue;
  }
}

hipError_t LaunchBlockMfma(const MfmaConfig& cfg, const MfmaParams& p, hipStream_t stream) {
  if (p.P == 0 || p.row_blocks == 0) return hipSuccess;
  if (p.ksteps > cfg.ks_max || p.ksteps > 32) return hipErrorInvalidValue;
  const size_t lds = (size_t)2 * p.ksteps * kMfmaTilePos * 16;
  if (lds > (size_t)kMaxLdsBytes) return hipErrorInvalidValue;
  const uint32_t tiles = (p.P + kMfmaTilePos - 1) / kMfmaTilePos;
  if (cfg.waves != 4) return hipErrorInvalidValue;
  MfmaParams q = p;
  q.tiles = (int)tiles;
  q.row_groups = (p.row_blocks + 3) / 4;
  dim3 grid(8u * q.row_groups * ((tiles + 7) / 8)), block(256);
  switch (cfg.out_kind) {
    case kOutF32:
      return MfmaByKs<kOutF32>(cfg, q, grid, block, lds, stream);
    case kOutI8:
      return MfmaByKs<kOutI8>(cfg, q, grid, block, lds, stream);
    case kOutAcc32:
      return MfmaByKs<kOutAcc32>(cfg, q, grid, block, lds, stream);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace pl
