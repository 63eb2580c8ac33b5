// Floor probes: what the device needs for the memory traffic and the launch of
// the metric shape's image kernel without any of its arithmetic.  Not part of
// the operator; bench.py --config floors times them next to the real kernel.
//
// All kernels use the image kernel's grid (one workgroup of 512 threads per
// image and 128 output rows, a contiguous range of items per XCD) unless noted.
//   0 empty          nothing
//   1 write          every workgroup writes its 128 output rows (fp32) as whole
//                    64-byte sectors, written through (sc1 nt)
//   2 stream         elementwise int8 -> fp32 over the same bytes, no
//                    dependence between positions (grid of 256-thread workgroups)
//   3 load           the image's activations are moved into LDS (direct
//                    global-to-LDS loads) and waited for
//   4 load + write   3, a barrier, then 1: the image kernel's memory schedule
//                    (no output byte can leave before every channel of its
//                    position has arrived) without transposition and multiply
//   5 load + transpose + write
//                    4 with the image kernel's in-place regrouping of the
//                    activations into matrix-core operand cells (4x4 byte
//                    transposes, LDS reads and writes) between load and barrier
#include <hip/hip_runtime.h>

#include <cstdint>

#include "launch_lds.h"

namespace {

typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

struct ProbeParams {
  const int8_t* x;
  char* out;
  int batch, ic, oc, hw;
  int row_groups, items, per_xcd;
};

__device__ __forceinline__ void StoreThrough(u4 v, void* p) { asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n s_nop 1" ::"v"(p), "v"(v) : "memory"); }

__device__ __forceinline__ bool Item(const ProbeParams& p, int* n, int* rg) {
  const int item = (int)(blockIdx.x & 7u) * p.per_xcd + (int)(blockIdx.x >> 3);
  if (item >= p.items) return false;
  *n = item / p.row_groups;
  *rg = item - *n * p.row_groups;
  return true;
}

// 128 rows x hw fp32 of image n: one contiguous piece of the output
__device__ __forceinline__ void WriteRows(const ProbeParams& p, int n, int rg, uint32_t seed) {
  char* base = p.out + ((size_t)n * p.oc + (size_t)rg * 128) * p.hw * 4;
  const int pieces = 128 * p.hw * 4 / 16;
  for (int i = threadIdx.x; i < pieces; i += blockDim.x) StoreThrough(u4{seed, (uint32_t)i, 2u, 3u}, base + (size_t)i * 16);
}

// the image's ic x hw bytes into LDS, 16 channels x hw bytes per wavefront and round
__device__ __forceinline__ void LoadImage(const ProbeParams& p, int n, char* lds) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int8_t* ximg = p.x + (size_t)n * p.ic * p.hw;
  const int blk = 16 * p.hw, full = blk / 1024, rem_lanes = (blk % 1024) / 16;
  for (int kg = wave; kg < p.ic / 16; kg += 8) {
    const int8_t* src = ximg + (size_t)kg * blk + lane * 16;
    char* dst = lds + (size_t)kg * blk;
    for (int t = 0; t < full; ++t)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + t * 1024), (__attribute__((address_space(3))) void*)(dst + t * 1024), 16, 0, 0);
    if (lane < rem_lanes)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + full * 1024), (__attribute__((address_space(3))) void*)(dst + full * 1024), 16, 0, 0);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// 4 dwords holding 4 channels x 4 positions -> 4 positions x 4 channels.
__device__ __forceinline__ void Transpose4x4(uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3) {
  const uint32_t a = __builtin_amdgcn_perm(r1, r0, 0x05010400u);
  const uint32_t b = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
  const uint32_t c = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
  const uint32_t d = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
  r0 = __builtin_amdgcn_perm(c, a, 0x05040100u);
  r1 = __builtin_amdgcn_perm(c, a, 0x07060302u);
  r2 = __builtin_amdgcn_perm(d, b, 0x05040100u);
  r3 = __builtin_amdgcn_perm(d, b, 0x07060302u);
}

__global__ void __launch_bounds__(512) EmptyKernel(const ProbeParams p) {
  int n, rg;
  if (!Item(p, &n, &rg)) return;
}

__global__ void __launch_bounds__(512) WriteKernel(const ProbeParams p) {
  int n, rg;
  if (!Item(p, &n, &rg)) return;
  WriteRows(p, n, rg, 1u);
}

__global__ void __launch_bounds__(256) StreamKernel(const ProbeParams p) {
  const size_t nvec = (size_t)p.batch * p.ic * p.hw / 16;  // 16 input bytes -> 64 output bytes
  const u4* x = reinterpret_cast<const u4*>(p.x);
  v4f* out = reinterpret_cast<v4f*>(p.out);
  const int lane = threadIdx.x & 63;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (size_t)gridDim.x * blockDim.x) {
    const u4 v = x[i];
    const size_t ob = 4 * (i - lane);  // the wavefront's 256 output vectors, 1 KB contiguous per store instruction
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint32_t w = v[c];
      const v4f o = {(float)(int8_t)(w & 255u), (float)(int8_t)((w >> 8) & 255u), (float)(int8_t)((w >> 16) & 255u), (float)(int8_t)(w >> 24)};
      __builtin_nontemporal_store(o, out + ob + c * 64 + lane);
    }
  }
}

__global__ void __launch_bounds__(512) LoadKernel(const ProbeParams p) {
  extern __shared__ uint4 lds[];
  int n, rg;
  if (!Item(p, &n, &rg)) return;
  LoadImage(p, n, reinterpret_cast<char*>(lds));
  __syncthreads();
  const uint32_t v = reinterpret_cast<const uint32_t*>(lds)[threadIdx.x];
  if (v == 0x5a5a5a5au && p.batch < 0) p.out[0] = 1;  // keeps the loads alive; never true
}

__global__ void __launch_bounds__(512) LoadWriteKernel(const ProbeParams p) {
  extern __shared__ uint4 lds[];
  int n, rg;
  if (!Item(p, &n, &rg)) return;
  LoadImage(p, n, reinterpret_cast<char*>(lds));
  __syncthreads();
  WriteRows(p, n, rg, reinterpret_cast<const uint32_t*>(lds)[threadIdx.x]);
}

__global__ void __launch_bounds__(512) LoadTransposeWriteKernel(const ProbeParams p) {
  extern __shared__ uint4 lds[];
  int n, rg;
  if (!Item(p, &n, &rg)) return;
  char* lbase = reinterpret_cast<char*>(lds);
  LoadImage(p, n, lbase);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int qpi = p.hw / 4;
  for (int kg = wave; kg < p.ic / 16; kg += 8) {
    uint32_t* blk = reinterpret_cast<uint32_t*>(lbase + (size_t)kg * 16 * p.hw);
    uint32_t r[16];
    if (lane < qpi) {
#pragma unroll
      for (int i = 0; i < 16; ++i) r[i] = blk[i * qpi + lane];
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_sched_barrier(0);
    if (lane < qpi) {
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) Transpose4x4(r[4 * b4], r[4 * b4 + 1], r[4 * b4 + 2], r[4 * b4 + 3]);
      uint4* cells = reinterpret_cast<uint4*>(blk) + lane;
#pragma unroll
      for (int c = 0; c < 4; ++c) cells[c * qpi] = make_uint4(r[c], r[4 + c], r[8 + c], r[12 + c]);
    }
  }
  __syncthreads();
  WriteRows(p, n, rg, reinterpret_cast<const uint32_t*>(lds)[threadIdx.x]);
}

}  // namespace

// kind as listed at the top.  x / out: `sets` buffers each, used in rotation;
// `launches` back-to-back launches on `stream`, their total time (HIP events on
// that stream) goes to *ms.  Returns 0, or a HIP error code.
extern "C" int pl_probe_floor(int kind, const void* const* x, void* const* out, int sets, int batch, int ic, int oc, int hw, int launches, void* stream, float* ms) {
  if (kind < 0 || kind > 5 || sets < 1 || batch < 1 || launches < 1 || ic % 16 != 0 || oc % 128 != 0 || hw % 4 != 0) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)ic * hw;
  if (kind >= 3 && lds > 160u * 1024u) return (int)hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  ProbeParams p{};
  p.batch = batch, p.ic = ic, p.oc = oc, p.hw = hw;
  p.row_groups = oc / 128;
  p.items = batch * p.row_groups;
  p.per_xcd = (p.items + 7) / 8;
  const dim3 grid(8u * (uint32_t)p.per_xcd), block(512);
  hipEvent_t e0, e1;
  hipError_t e = hipEventCreate(&e0);
  if (e != hipSuccess) return (int)e;
  e = hipEventCreate(&e1);
  if (e != hipSuccess) return (int)e;
  e = hipEventRecord(e0, s);
  for (int i = 0; i < launches && e == hipSuccess; ++i) {
    p.x = static_cast<const int8_t*>(x[i % sets]);
    p.out = static_cast<char*>(out[i % sets]);
    switch (kind) {
      case 0:
        e = pl::LaunchWithLds(EmptyKernel, grid, block, 0, s, p);
        break;
      case 1:
        e = pl::LaunchWithLds(WriteKernel, grid, block, 0, s, p);
        break;
      case 2:
        e = pl::LaunchWithLds(StreamKernel, dim3(2048), dim3(256), 0, s, p);
        break;
      case 3:
        e = pl::LaunchWithLds(LoadKernel, grid, block, lds, s, p);
        break;
      case 4:
        e = pl::LaunchWithLds(LoadWriteKernel, grid, block, lds, s, p);
        break;
      default:
        e = pl::LaunchWithLds(LoadTransposeWriteKernel, grid, block, lds, s, p);
        break;
    }
  }
  if (e == hipSuccess) e = hipEventRecord(e1, s);
  if (e == hipSuccess) e = hipEventSynchronize(e1);
  float t = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&t, e0, e1);
  if (ms) *ms = t;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return (int)e;
}
