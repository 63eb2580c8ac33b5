// Launch helper shared by the kernel files: dynamic LDS above the default
// limit has to be enabled per kernel function and device before the launch.
#pragma once

#include <hip/hip_runtime.h>

#include <map>
#include <mutex>
#include <utility>

namespace pl {

// Remembers, per (kernel function, device), the largest dynamic LDS size
// already enabled.  Keyed on the function's address: instantiations of one
// kernel template share a function *type* but not an address.  May be called
// from any thread.
inline hipError_t EnableDynamicLds(const void* kernel, size_t lds) {
  if (lds <= 48 * 1024) return hipSuccess;
  static std::mutex mu;
  static std::map<std::pair<const void*, int>, size_t> enabled;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(mu);
  size_t& have = enabled[std::make_pair(kernel, dev)];
  if (have >= lds) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
  if (e == hipSuccess) have = lds;
  return e;
}

template <typename Kernel, typename... Args>
hipError_t LaunchWithLds(Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const Args&... args) {
  const hipError_t e = EnableDynamicLds(reinterpret_cast<const void*>(kernel), lds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kernel, grid, block, lds, stream, args...);
  return hipGetLastError();
}

}  // namespace pl
