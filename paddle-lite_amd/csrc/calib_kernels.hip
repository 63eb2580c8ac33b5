// Precision-change kernels around the int8 sparse convolution: fp32 -> int8
// with a per-tensor scale and back.  Pure streaming work with fully
// coalesced accesses, a scalar head and tail for buffers that are not 16-byte
// aligned or whose length is not a multiple of four.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "sparse_conv_kernels.h"

namespace pl {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));

// max(v, -127), round half away from zero, min(., 127): clamp first (the
// bounds are integers), then truncate the sum with the largest float below
// one half.
__device__ __forceinline__ int QuantizeI8(float v) {
  v = __builtin_amdgcn_fmed3f(v, -127.0f, 127.0f);
  return static_cast<int>(v + __builtin_copysignf(0x1.fffffep-2f, v));
}

__device__ __forceinline__ uint32_t PackI8x4(int a, int b, int c, int d) {
  const uint32_t ab = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
  const uint32_t cd = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
  return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

// Work is cut into units of four elements; lane l of a wavefront takes unit
// base + l, so the 16-byte side of every access is 1 KB contiguous per
// instruction and the 4-byte side 256 B.  A thread has four units in flight.
// `head` elements (0..3, up to where the 16-byte side is aligned) and the
// elements after the last full unit are done one by one by the first
// workgroup.  The 4-byte side may sit at any byte address: global memory
// takes dword accesses unaligned.
constexpr int kUnroll = 4;

__global__ void __launch_bounds__(256) Fp32ToInt8Kernel(const float* __restrict__ x, int8_t* __restrict__ out, int64_t n, float inv_scale, int64_t head, int64_t units) {
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  const v4f* xb = reinterpret_cast<const v4f*>(x + head);
  uint32_t* ob = reinterpret_cast<uint32_t*>(out + head);
  for (int64_t u0 = tid; u0 < units; u0 += kUnroll * nthreads) {
    v4f v[kUnroll];
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
      const int64_t u = u0 + i * nthreads;
      v[i] = __builtin_nontemporal_load(xb + (u < units ? u : u0));
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
      const int64_t u = u0 + i * nthreads;
      const uint32_t w = PackI8x4(QuantizeI8(v[i].x * inv_scale), QuantizeI8(v[i].y * inv_scale), QuantizeI8(v[i].z * inv_scale), QuantizeI8(v[i].w * inv_scale));
      if (u < units) __builtin_nontemporal_store(w, ob + u);
    }
  }
  if (blockIdx.x == 0) {
    const int64_t tail0 = head + units * 4;
    for (int64_t i = threadIdx.x; i < head; i += blockDim.x) out[i] = static_cast<int8_t>(QuantizeI8(x[i] * inv_scale));
    for (int64_t i = tail0 + threadIdx.x; i < n; i += blockDim.x) out[i] = static_cast<int8_t>(QuantizeI8(x[i] * inv_scale));
  }
}

__global__ void __launch_bounds__(256) Int8ToFp32Kernel(const int8_t* __restrict__ x, float* __restrict__ out, int64_t n, float scale, int64_t head, int64_t units) {
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  const int* xb = reinterpret_cast<const int*>(x + head);
  v4f* ob = reinterpret_cast<v4f*>(out + head);
  for (int64_t u0 = tid; u0 < units; u0 += kUnroll * nthreads) {
    int d[kUnroll];
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
      const int64_t u = u0 + i * nthreads;
      d[i] = __builtin_nontemporal_load(xb + (u < units ? u : u0));
    }
#pragma unroll
    for (int i = 0; i < kUnroll; ++i) {
      const int64_t u = u0 + i * nthreads;
      v4f v;
      v.x = (float)(int8_t)(d[i] & 0xff) * scale;
      v.y = (float)(int8_t)((d[i] >> 8) & 0xff) * scale;
      v.z = (float)(int8_t)((d[i] >> 16) & 0xff) * scale;
      v.w = (float)(d[i] >> 24) * scale;
      if (u < units) __builtin_nontemporal_store(v, ob + u);
    }
  }
  if (blockIdx.x == 0) {
    const int64_t tail0 = head + units * 4;
    for (int64_t i = threadIdx.x; i < head; i += blockDim.x) out[i] = (float)x[i] * scale;
    for (int64_t i = tail0 + threadIdx.x; i < n; i += blockDim.x) out[i] = (float)x[i] * scale;
  }
}

// Grid: one pass of kUnroll units per thread, capped (the loop strides over
// the rest).
unsigned GridFor(int64_t units) {
  const int64_t wgs = (units + 256 * kUnroll - 1) / (256 * kUnroll);
  return (unsigned)(wgs < 1 ? 1 : (wgs > 16384 ? 16384 : wgs));
}

}  // namespace

hipError_t LaunchFp32ToInt8(const float* x, int8_t* out, int64_t n, float scale, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  // the 16-byte loads start where the input is 16-byte aligned
  int64_t head = (int64_t)(((16 - (reinterpret_cast<uintptr_t>(x) & 15)) & 15) / 4);
  if (head > n) head = n;
  const int64_t units = (n - head) / 4;
  // 1.f / scale first, then one multiply per element, as the reference does
  const float inv_scale = 1.0f / scale;
  hipLaunchKernelGGL(Fp32ToInt8Kernel, dim3(GridFor(units)), dim3(256), 0, stream, x, out, n, inv_scale, head, units);
  return hipGetLastError();
}

hipError_t LaunchInt8ToFp32(const int8_t* x, float* out, int64_t n, float scale, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  // the 16-byte stores start where the output is 16-byte aligned
  int64_t head = (int64_t)(((16 - (reinterpret_cast<uintptr_t>(out) & 15)) & 15) / 4);
  if (head > n) head = n;
  const int64_t units = (n - head) / 4;
  hipLaunchKernelGGL(Int8ToFp32Kernel, dim3(GridFor(units)), dim3(256), 0, stream, x, out, n, scale, head, units);
  return hipGetLastError();
}

}  // namespace pl
