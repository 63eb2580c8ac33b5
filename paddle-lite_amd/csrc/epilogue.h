// Epilogue arithmetic shared by the kernels of this library: activation,
// int8 quantisation and byte packing, as device inline functions.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "sparse_conv_kernels.h"

namespace pl {
namespace epilogue {

// min(max(v, 0), hi) for any hi as one median instruction: the lower bound
// min(0, hi) is wave-uniform and makes the median equal hi when hi < 0.
__device__ __forceinline__ float Clamp0(float v, float hi) { return __builtin_amdgcn_fmed3f(v, fminf(0.0f, hi), hi); }

__device__ __forceinline__ float Activate(float v, const DevAct& a) {
  switch (a.type) {
    case 1:
      return fmaxf(v, 0.0f);
    case 2:
      return Clamp0(v, a.relu6_coef);
    case 4:
      return (v >= 0.0f) ? v : v * a.leaky_alpha;
    case 10:
      return (v * a.hs_inv_scale) * Clamp0(v + a.hs_offset, a.hs_threshold);
    default:
      return v;
  }
}

// Same, with the activation fixed at compile time; DispatchAct turns the
// run-time type into that constant once per kernel instead of once per value.
// Not a PL_ACT_* value: what a kernel may dispatch on instead of leaky_relu (4) when 0 < slope <= 1.
constexpr int kActLeakyUnitSlope = 5;
__device__ __forceinline__ int LeakyAsMax(const DevAct& a) { return a.type == 4 && a.leaky_alpha > 0.0f && a.leaky_alpha <= 1.0f ? kActLeakyUnitSlope : a.type; }

template <int ACT>
__device__ __forceinline__ float ActivateT(float v, const DevAct& a) {
  if (ACT == 1) return fmaxf(v, 0.0f);
  if (ACT == 2) return Clamp0(v, a.relu6_coef);
  if (ACT == 4) return (v >= 0.0f) ? v : v * a.leaky_alpha;
  // leaky_relu with a slope in (0, 1]: the larger of v and slope * v is the same value for every v (zeros keep
  // their sign, infinities stay, a NaN stays a NaN) in two instructions instead of three
  if (ACT == kActLeakyUnitSlope) return __builtin_fmaxf(v, v * a.leaky_alpha);
  if (ACT == 10) return (v * a.hs_inv_scale) * Clamp0(v + a.hs_offset, a.hs_threshold);
  return v;
}

template <typename F>
__device__ __forceinline__ void DispatchAct(int type, F&& f) {
  switch (type) {
    case kActLeakyUnitSlope:
      f(std::integral_constant<int, kActLeakyUnitSlope>());
      break;
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

// max(v, -127), round half away from zero, min(., 127).  The bounds are
// integers, so clamping first gives the same result; rounding half away from
// zero is the truncated sum with the largest float below one half (adding one
// half itself would carry 0.49999997 up to 1).  QuantizeF is that sum, the
// float whose truncation is the int8 value.
__device__ __forceinline__ float QuantizeF(float v) {
  v = __builtin_amdgcn_fmed3f(v, -127.0f, 127.0f);
  return v + __builtin_copysignf(0x1.fffffep-2f, v);
}
__device__ __forceinline__ int QuantizeI8(float v) { return static_cast<int>(QuantizeF(v)); }

// Activation and quantisation of one value, up to the truncation.  relu
// followed by the clamp is one median, and its result has no sign to copy.
template <int ACT>
__device__ __forceinline__ float ActQuantF(float v, const DevAct& a) {
  if (ACT == 1) return __builtin_amdgcn_fmed3f(v, 0.0f, 127.0f) + 0x1.fffffep-2f;
  if (ACT == 2) {
    // relu6 followed by the clamp is one median over the intersected bounds
    // (wave-uniform, computed once), and the sign of its result is the sign
    // of the coefficient: [0, coef] for coef >= 0, the constant coef below.
    const float hi = a.relu6_coef;
    const float lo127 = fmaxf(fminf(0.0f, hi), -127.0f);
    const float hi127 = fmaxf(fminf(hi, 127.0f), lo127);
    const float half = hi >= 0.0f ? 0x1.fffffep-2f : -0x1.fffffep-2f;
    return __builtin_amdgcn_fmed3f(v, lo127, hi127) + half;
  }
  if (ACT < 0) return QuantizeF(Activate(v, a));
  return QuantizeF(ActivateT<(ACT < 0 ? 0 : ACT)>(v, a));
}
template <int ACT>
__device__ __forceinline__ int ActQuantI8(float v, const DevAct& a) {
  return static_cast<int>(ActQuantF<ACT>(v, a));
}

// Truncates eight floats to integers and packs their low bytes into two
// dwords (a0 in byte 0 of the first).  The conversion writes its byte straight
// into the destination register (sub-dword destination select), so no separate
// packing instruction is needed.  An instruction that writes part of a
// register must not be followed directly by one that reads that register: the
// two dwords are filled alternately and a wait state closes the sequence.
__device__ __forceinline__ void TruncPackI8x8(float a0, float a1, float a2, float a3, float b0, float b1, float b2, float b3, uint32_t& a, uint32_t& b) {
  asm("v_cvt_i32_f32_sdwa %0, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
      "v_cvt_i32_f32_sdwa %1, %6 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
      "v_cvt_i32_f32_sdwa %0, %3 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "v_cvt_i32_f32_sdwa %1, %7 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "v_cvt_i32_f32_sdwa %0, %4 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "v_cvt_i32_f32_sdwa %1, %8 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "v_cvt_i32_f32_sdwa %0, %5 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "v_cvt_i32_f32_sdwa %1, %9 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "s_nop 0"
      : "=&v"(a), "=&v"(b)
      : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b0), "v"(b1), "v"(b2), "v"(b3));
}

// The same for four floats and one dword; a wait state separates each
// conversion from the next one, which reads the register it completes.
__device__ __forceinline__ uint32_t TruncPackI8x4(float a0, float a1, float a2, float a3) {
  uint32_t a;
  asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD\n\t"
      "s_nop 0\n\t"
      "v_cvt_i32_f32_sdwa %0, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "s_nop 0\n\t"
      "v_cvt_i32_f32_sdwa %0, %3 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "s_nop 0\n\t"
      "v_cvt_i32_f32_sdwa %0, %4 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD\n\t"
      "s_nop 0"
      : "=&v"(a)
      : "v"(a0), "v"(a1), "v"(a2), "v"(a3));
  return a;
}

// Low bytes of four quantized values as one dword (a in byte 0).
__device__ __forceinline__ uint32_t PackI8x4(int a, int b, int c, int d) {
  // perm(hi, lo, sel): selector 0-3 = byte of lo, 4-7 = byte of hi, 0x0c = zero
  const uint32_t ab = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
  const uint32_t cd = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
  return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

}  // namespace epilogue
}  // namespace pl
