// Floor probes: what the device needs for the memory traffic and the launch of
// the metric shape's image kernel without any of its arithmetic.  Not part of
// the operator (a library of its own, built from this file alone);
// bench.py --config floors times them next to the real kernel,
// bench.py --config store-shapes times the store patterns at the end of this
// file, and tests/test_gpu_lds_transpose.py checks the lane mapping of the
// transposing LDS read that the image kernels rely on.
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
//   6 load + regroup by transposing reads + write
//                    5 with the regrouping done by ds_read_b64_tr_b8 and
//                    16-byte LDS writes (512 channels, 14 x 14 only)
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../paddle-lite_amd/csrc/launch_lds.h"

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

// 6: the regrouping of image_mfma_kernels.hip's TRG variant (64 channel rows per wavefront, cells of 16
// channels of one parity, four apart), without the padding between cell groups
__global__ void __launch_bounds__(512) LoadTrRegroupWriteKernel(const ProbeParams p) {
  extern __shared__ uint4 lds[];
  typedef int v2i __attribute__((ext_vector_type(2)));
  typedef int v4i __attribute__((ext_vector_type(4)));
  int n, rg;
  if (!Item(p, &n, &rg)) return;
  char* lbase = reinterpret_cast<char*>(lds) + 256;
  LoadImage(p, n, lbase);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int hw = p.hw, qpi = hw / 4;
  auto reg = (__attribute__((address_space(3))) char*)lbase + wave * 64 * hw;
  const int g = lane >> 4, s16 = lane & 15, par = g >> 1;
  const int rbase = (4 * (8 * (g & 1) + (s16 >> 1)) + par) * hw + 8 * (s16 & 1) - 4 * par;
  v2i rr[13][2];
#pragma unroll
  for (int i = 0; i < 13; ++i)
#pragma unroll
    for (int r2 = 0; r2 < 2; ++r2) rr[i][r2] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<__attribute__((address_space(3))) v2i*>(reg + rbase + 16 * i + 2 * r2 * hw));
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_sched_barrier(0);
  auto cells = reinterpret_cast<__attribute__((address_space(3))) v4i*>(reg + g * 16 * hw);
#pragma unroll
  for (int i = 0; i < 13; ++i) {
    const int pos = 16 * i - 4 * par + s16;
    if (pos >= 0 && pos < hw) cells[(pos & 3) * qpi + (pos >> 2)] = v4i{rr[i][0].x, rr[i][0].y, rr[i][1].x, rr[i][1].y};
  }
  __syncthreads();
  WriteRows(p, n, rg, reinterpret_cast<const uint32_t*>(lds)[64 + threadIdx.x]);
}

// Lane mapping of ds_read_b64_tr_b8: LDS byte i holds i (low byte in pass 0, high byte in pass 1), lane l
// reads at addr[l]; out[l][0..1] = the two dwords it receives.
__global__ void Tr8MapKernel(uint32_t* out, const int* addr, int pass) {
  extern __shared__ uint4 lds[];
  typedef int v2i __attribute__((ext_vector_type(2)));
  char* bytes = reinterpret_cast<char*>(lds);
  for (int i = threadIdx.x; i < 4096; i += blockDim.x) bytes[i] = pass == 0 ? (char)(i & 0xff) : (char)(i >> 8);
  __syncthreads();
  auto l3 = (__attribute__((address_space(3))) char*)bytes;
  const v2i v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(reinterpret_cast<__attribute__((address_space(3))) v2i*>(l3 + addr[threadIdx.x]));
  out[2 * threadIdx.x] = (uint32_t)v.x;
  out[2 * threadIdx.x + 1] = (uint32_t)v.y;
}

// Store patterns over the fp32 output of the metric shape (every workgroup writes its 128 rows x 196
// floats, a wavefront the 16 rows rho + 4 (16 j + n) of the image kernels):
//   0  an instruction writes 16 rows x 64 bytes (one sector of every row), sectors in order
//   1  an instruction writes 4 rows x 256 bytes starting on sector boundaries (the regrouping image kernel)
//   2  an instruction writes 8 rows x 128 bytes, whole lines (the kernel with transposing reads)
// POL 0: sc1 nt (written through), 1: nt, 2: plain
typedef uint32_t su4 __attribute__((ext_vector_type(4)));
template <int POL>
__device__ __forceinline__ void ShapeStore(su4 v, char* base, uint32_t off) {
  if (POL == 0) asm volatile("global_store_dwordx4 %0, %1, %2 sc1 nt\n s_nop 1" ::"v"(off), "v"(v), "s"(base) : "memory");
  if (POL == 1) asm volatile("global_store_dwordx4 %0, %1, %2 nt\n s_nop 1" ::"v"(off), "v"(v), "s"(base) : "memory");
  if (POL == 2) asm volatile("global_store_dwordx4 %0, %1, %2\n s_nop 1" ::"v"(off), "v"(v), "s"(base) : "memory");
}
template <int MODE, int POL>
__global__ void __launch_bounds__(512) StoreShapeKernel(char* out) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int item = (int)(blockIdx.x & 7u) * 32 + (int)(blockIdx.x >> 3);
  char* base = out + (size_t)item * 128 * 784;
  const int rho = wave & 3, j = wave >> 2, n = lane & 15, kq = lane >> 4;
  const su4 v = su4{(uint32_t)lane, (uint32_t)wave, 3u, 4u};
  if (MODE == 0) {
    const int row = rho + 4 * (16 * j + n);
    const int a0 = (16 - 4 * (row & 3)) & 15;  // positions to the first sector boundary of the row
    for (int t = 0; t < 13; ++t) {
      const int first = a0 + 16 * ((a0 > 0 ? -1 : 0) + t), pos = first + 4 * kq;
      if (pos >= 0 && pos < 196) {
        if (first >= 0 && first + 16 <= 196) ShapeStore<POL>(v, base, (uint32_t)(row * 784 + pos * 4));
        else *reinterpret_cast<su4*>(base + row * 784 + pos * 4) = v;
      }
    }
  } else if (MODE == 1) {
    for (int t = 0; t < 13; ++t) {
      const int rgrp = t & 3, piece = t >> 2;  // 4 groups of 4 rows x 3 full pieces, then the leftovers
      const int row = rho + 4 * (16 * j + 4 * rgrp + kq);
      const int aq = (4 - (row & 3)) & 3;       // quads to the first sector boundary
      if (t < 12) {
        ShapeStore<POL>(v, base, (uint32_t)(row * 784 + (aq + 16 * piece + n) * 16));
      } else {
        for (int r2 = 0; r2 < 4; ++r2) {
          const int row2 = rho + 4 * (16 * j + 4 * r2 + kq);
          const int aq2 = (4 - (row2 & 3)) & 3;
          const int qq = n < aq2 ? n : aq2 + 48 + (n - aq2);
          if (qq < 49) *reinterpret_cast<su4*>(base + row2 * 784 + qq * 16) = v;
        }
      }
    }
  } else {
    const int piece = lane & 7, m = lane >> 3;
    for (int t = 0; t < 14; ++t) {
      const int row = rho + 4 * (16 * j + 2 * m + (t & 1));
      const int a0 = (32 - 4 * (row & 7)) & 31;  // positions to the first line boundary of the row
      const int first = a0 + 32 * ((a0 > 0 ? -1 : 0) + (t >> 1)), pos = first + 4 * piece;
      if (pos >= 0 && pos < 196) {
        if (first >= 0 && first + 32 <= 196) ShapeStore<POL>(v, base, (uint32_t)(row * 784 + pos * 4));
        else *reinterpret_cast<su4*>(base + row * 784 + pos * 4) = v;
      }
    }
  }
}

template <int MODE>
hipError_t LaunchShape(int pol, char* out, hipStream_t s) {
  if (pol == 0) hipLaunchKernelGGL((StoreShapeKernel<MODE, 0>), dim3(256), dim3(512), 0, s, out);
  else if (pol == 1) hipLaunchKernelGGL((StoreShapeKernel<MODE, 1>), dim3(256), dim3(512), 0, s, out);
  else hipLaunchKernelGGL((StoreShapeKernel<MODE, 2>), dim3(256), dim3(512), 0, s, out);
  return hipGetLastError();
}

}  // namespace

// kind as listed at the top.  x / out: `sets` buffers each, used in rotation;
// `launches` back-to-back launches on `stream`, their total time (HIP events on
// that stream) goes to *ms.  Returns 0, or a HIP error code.
extern "C" int pl_probe_floor(int kind, const void* const* x, void* const* out, int sets, int batch, int ic, int oc, int hw, int launches, void* stream, float* ms) {
  if (kind < 0 || kind > 6 || sets < 1 || batch < 1 || launches < 1 || ic % 16 != 0 || oc % 128 != 0 || hw % 4 != 0) return (int)hipErrorInvalidValue;
  // what the kernels assume: the stream probe writes ic x hw floats per image into an oc x hw buffer, the
  // load probes read 2 KB of the staged image back, the transposing ones hold a position quad per lane
  if (kind == 2 && ic > oc) return (int)hipErrorInvalidValue;
  if (kind >= 3 && (size_t)ic * hw < 2048) return (int)hipErrorInvalidValue;
  if (kind == 5 && hw > 256) return (int)hipErrorInvalidValue;
  if (kind == 6 && (ic != 512 || hw != 196)) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)ic * hw + (kind == 6 ? 512 : 0);
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
  if (e != hipSuccess) {
    (void)hipEventDestroy(e0);
    return (int)e;
  }
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
      case 5:
        e = pl::LaunchWithLds(LoadTransposeWriteKernel, grid, block, lds, s, p);
        break;
      default:
        e = pl::LaunchWithLds(LoadTrRegroupWriteKernel, grid, block, lds, s, p);
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

// The lane mapping of ds_read_b64_tr_b8: lane l reads at LDS byte offset addr[l] (64 entries, below 4088);
// src[8 l + b] = LDS byte offset that byte b of lane l's result came from.  Host pointers.  Returns 0 or a
// HIP error code.
extern "C" int pl_probe_tr8_map(const int* addr, uint16_t* src) {
  for (int l = 0; l < 64; ++l)
    if (addr[l] < 0 || addr[l] > 4088) return (int)hipErrorInvalidValue;
  int* daddr = nullptr;
  uint32_t* dout = nullptr;
  hipError_t e = hipMalloc(&daddr, 64 * sizeof(int));
  if (e == hipSuccess) e = hipMalloc(&dout, 128 * sizeof(uint32_t));
  if (e == hipSuccess) e = hipMemcpy(daddr, addr, 64 * sizeof(int), hipMemcpyHostToDevice);
  uint32_t lo[128], hi[128];
  for (int pass = 0; pass < 2 && e == hipSuccess; ++pass) {
    hipLaunchKernelGGL(Tr8MapKernel, dim3(1), dim3(64), 4096, 0, dout, daddr, pass);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpy(pass == 0 ? lo : hi, dout, sizeof(lo), hipMemcpyDeviceToHost);
  }
  if (e == hipSuccess) {
    for (int l = 0; l < 64; ++l)
      for (int b = 0; b < 8; ++b) src[8 * l + b] = (uint16_t)(((lo[2 * l + b / 4] >> (8 * (b % 4))) & 0xffu) | (((hi[2 * l + b / 4] >> (8 * (b % 4))) & 0xffu) << 8));
  }
  if (daddr) (void)hipFree(daddr);
  if (dout) (void)hipFree(dout);
  return (int)e;
}

// `launches` back-to-back launches of store pattern `mode` with policy `pol` (see StoreShapeKernel) over
// the 64 x 512 x 196 fp32 buffers out[0 .. sets - 1] in rotation; total time in *ms.
extern "C" int pl_probe_store_shape(int mode, int pol, void* const* out, int sets, int launches, void* stream, float* ms) {
  if (mode < 0 || mode > 2 || pol < 0 || pol > 2 || sets < 1 || launches < 1) return (int)hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipEvent_t e0, e1;
  hipError_t e = hipEventCreate(&e0);
  if (e != hipSuccess) return (int)e;
  e = hipEventCreate(&e1);
  if (e != hipSuccess) {
    (void)hipEventDestroy(e0);
    return (int)e;
  }
  e = hipEventRecord(e0, s);
  for (int i = 0; i < launches && e == hipSuccess; ++i) {
    char* o = static_cast<char*>(out[i % sets]);
    e = mode == 0 ? LaunchShape<0>(pol, o, s) : (mode == 1 ? LaunchShape<1>(pol, o, s) : LaunchShape<2>(pol, o, s));
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
