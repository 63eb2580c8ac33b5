// Kernel arguments in registers.  A kernel that takes its parameters as one by-value struct finds them in the
// kernel-argument segment and starts with a load from memory that everything else waits for.  The leading
// scalar arguments of a kernel can instead be handed to every wavefront in registers when it starts
// (kernel-argument preload, -amdgpu-kernarg-preload-count in the build; up to 14 dwords).  The helpers here
// pass the first 56 bytes of a parameter block a second time, as seven leading pointer-sized arguments, and
// put them back over the block inside the kernel: fields in that head are then read from registers, the rest
// from the block as before.  Blocks keep the pointers and sizes that the first loads of a kernel need in
// their first 56 bytes.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstring>
#include <type_traits>

#include "launch_lds.h"

namespace pl {

constexpr int kHeadWords = 7;

#define PL_HEAD_PARAMS                                                                                              \
  const void *pl_h0, const void *pl_h1, const void *pl_h2, const void *pl_h3, const void *pl_h4, const void *pl_h5, \
      const void *pl_h6
#define PL_HEAD_ARGS pl_h0, pl_h1, pl_h2, pl_h3, pl_h4, pl_h5, pl_h6

// The block with its first 56 bytes taken from the leading arguments.
template <typename P>
__device__ __forceinline__ P WithHead(const P& block, PL_HEAD_PARAMS) {
  static_assert(std::is_trivially_copyable<P>::value && sizeof(P) >= kHeadWords * 8 && alignof(P) == 8, "parameter block with an 8-byte aligned head");
  P p = block;
  const void* h[kHeadWords] = {PL_HEAD_ARGS};
  __builtin_memcpy(&p, h, sizeof(h));
  return p;
}

// Compile-time check that a field lies inside the head: PL_IN_HEAD(ImageMfmaParams, qpi).
#define PL_IN_HEAD(Block, field) \
  static_assert(offsetof(Block, field) + sizeof(Block::field) <= ::pl::kHeadWords * 8, #field " must lie in the first 56 bytes of " #Block)

// Launches kernel(head words..., block, further arguments...).
template <typename Kernel, typename P, typename... More>
hipError_t LaunchWithHead(Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const P& p, const More&... more) {
  static_assert(std::is_trivially_copyable<P>::value && sizeof(P) >= kHeadWords * 8 && alignof(P) == 8, "parameter block with an 8-byte aligned head");
  const void* h[kHeadWords];
  std::memcpy(h, &p, sizeof(h));
  return LaunchWithLds(kernel, grid, block, lds, stream, h[0], h[1], h[2], h[3], h[4], h[5], h[6], p, more...);
}

}  // namespace pl
