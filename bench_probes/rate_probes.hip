// Instruction-rate probes of one CU (gfx950): LDS reads and writes by width and pattern, the int8 matrix instruction,
// fp32 fused multiply-add, and the two interleaved.  One workgroup per CU (256 workgroups), every wavefront times its
// own loop with s_memtime and s_memrealtime (100 MHz); the host takes medians.  Built into bench_probes/libpl_probe.so
// next to the floor probes; bench.py --config device-rates prints the table.  Nothing of the operator links this.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
#define PL_LDS __attribute__((address_space(3)))

constexpr int kReps = 8, kPerRep = 64;  // LDS: instructions per wavefront = kReps * kPerRep

// LDS modes: 0 ds_read_b128 contiguous, 1 ds_read_b64, 2 ds_read_b32, 3 ds_read_b64_tr_b8, 4 ds_write_b128,
// 5 ds_write_b64, 6 ds_read_b128 as the image kernels read operand cells (16 cells per quarter wavefront, quarters
// 3328 bytes apart), 7 the same with quarters 3392 bytes apart
template <int MODE>
__global__ void __launch_bounds__(512) LdsRate(unsigned long long* out, int* sink) {
  extern __shared__ char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  PL_LDS char* base = (PL_LDS char*)lds + wave * 8192;
  for (int i = threadIdx.x; i < 65536 / 4; i += 512) ((int*)lds)[i] = i;
  __syncthreads();
  v4i acc = {0, 0, 0, 0};
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  for (int r = 0; r < kReps; ++r) {
#pragma unroll
    for (int j = 0; j < kPerRep / 8; ++j) {
      asm volatile("" ::: "memory");  // the eight accesses of a batch are not merged with those of the next
      if (MODE == 0 || MODE == 6 || MODE == 7) {
        v4i v[8];
        PL_LDS char* b = MODE == 0 ? base + lane * 16 : (PL_LDS char*)lds + (wave & 1) * 784 + (lane & 15) * 16 + (lane >> 4) * (MODE == 6 ? 3328 : 3392);
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = *(PL_LDS v4i*)(b + (MODE == 0 ? u * 1024 : (u & 3) * 13312 + (u >> 2) * 784));
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
      } else if (MODE == 1 || MODE == 3) {
        v2i v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          v[u] = MODE == 1 ? *(PL_LDS v2i*)(base + u * 1024 + lane * 8) : __builtin_amdgcn_ds_read_tr8_b64_v2i32((PL_LDS v2i*)(base + u * 1024 + lane * 8));
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          acc.x += v[u].x;
          acc.y += v[u].y;
        }
      } else if (MODE == 2) {
        int v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = *(PL_LDS int*)(base + u * 1024 + lane * 4);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc.x += v[u];
      } else if (MODE == 4) {
#pragma unroll
        for (int u = 0; u < 8; ++u) *(PL_LDS v4i*)(base + u * 1024 + lane * 16) = acc + (j * 8 + u);
      } else {
#pragma unroll
        for (int u = 0; u < 8; ++u) *(PL_LDS v2i*)(base + u * 1024 + lane * 8) = v2i{acc.x + j * 8 + u, acc.y};
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  __syncthreads();
  const unsigned long long t2 = __builtin_amdgcn_s_memtime();
  if (acc.x == 0x7fffffff) sink[0] = acc.y + acc.z + acc.w;
  if (lane == 0) {
    out[(blockIdx.x * 8 + wave) * 2] = t1 - t0;
    out[(blockIdx.x * 8 + wave) * 2 + 1] = t2 - t0;  // until the slowest wavefront of the workgroup is through
  }
}

// ALU modes: 0 eight independent matrix instructions per iteration, 1 a dependent chain of eight, 2 eight independent
// fp32 fused multiply-adds, 3 four matrix instructions with two multiply-adds behind each
constexpr int kAluIters = 256;
template <int MODE, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) AluRate(unsigned long long* out, int* sink, int seed) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const v4i a = {seed + lane, seed, lane, 3}, b = {lane, seed * 3, 7, lane * seed};
  v4i acc[8];
  float f[8];
  for (int i = 0; i < 8; ++i) {
    acc[i] = v4i{i, i, i, i};
    f[i] = (float)(lane + i);
  }
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int r = 0; r < kAluIters; ++r) {
    if (MODE == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[i], 0, 0, 0);
    } else if (MODE == 1) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[0], 0, 0, 0);
    } else if (MODE == 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = __builtin_fmaf(f[i], 1.0001f, 0.5f);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[i], 0, 0, 0);
        f[2 * i] = __builtin_fmaf(f[2 * i], 1.0001f, 0.5f);
        f[2 * i + 1] = __builtin_fmaf(f[2 * i + 1], 1.0001f, 0.5f);
      }
    }
  }
  int s = 0;
  for (int i = 0; i < 8; ++i) s += acc[i].x + acc[i].y + acc[i].z + acc[i].w + (int)f[i];
  const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if (s == 0x7fffffff) sink[0] = s;
  if (lane == 0) {
    out[(blockIdx.x * WAVES + wave) * 2] = t1 - t0;
    out[(blockIdx.x * WAVES + wave) * 2 + 1] = r1 - r0;
  }
}

template <int MODE>
hipError_t LaunchLds(unsigned long long* out, int* sink, hipStream_t s) {
  hipLaunchKernelGGL(LdsRate<MODE>, dim3(256), dim3(512), 65536, s, out, sink);
  return hipGetLastError();
}
template <int MODE>
hipError_t LaunchAlu(int waves, unsigned long long* out, int* sink, hipStream_t s) {
  if (waves == 4) hipLaunchKernelGGL((AluRate<MODE, 4>), dim3(256), dim3(256), 0, s, out, sink, 5);
  else hipLaunchKernelGGL((AluRate<MODE, 8>), dim3(256), dim3(512), 0, s, out, sink, 5);
  return hipGetLastError();
}

}  // namespace

// One launch of an LDS probe (mode 0 .. 7, see LdsRate).  out_dev: 256 x 8 x 2 counters (device memory): per wavefront
// the s_memtime counts of its own accesses and of the workgroup's slowest; sink_dev: one int.  Returns a HIP error code;
// *bytes_per_wavefront is what a wavefront moved.
extern "C" int pl_probe_lds_rate(int mode, unsigned long long* out_dev, int* sink_dev, void* stream, long long* bytes_per_wavefront) {
  if (!out_dev || !sink_dev || !bytes_per_wavefront || mode < 0 || mode > 7) return (int)hipErrorInvalidValue;
  static const int width[8] = {16, 8, 4, 8, 16, 8, 16, 16};
  *bytes_per_wavefront = (long long)kReps * kPerRep * 64 * width[mode];
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e = hipSuccess;
  switch (mode) {
    case 0: e = LaunchLds<0>(out_dev, sink_dev, s); break;
    case 1: e = LaunchLds<1>(out_dev, sink_dev, s); break;
    case 2: e = LaunchLds<2>(out_dev, sink_dev, s); break;
    case 3: e = LaunchLds<3>(out_dev, sink_dev, s); break;
    case 4: e = LaunchLds<4>(out_dev, sink_dev, s); break;
    case 5: e = LaunchLds<5>(out_dev, sink_dev, s); break;
    case 6: e = LaunchLds<6>(out_dev, sink_dev, s); break;
    default: e = LaunchLds<7>(out_dev, sink_dev, s); break;
  }
  return (int)e;
}

// One launch of an ALU probe (mode 0 .. 3, see AluRate) with 4 or 8 wavefronts per workgroup (1 or 2 per SIMD).
// out_dev: 256 x waves x 2 counters: s_memtime counts and s_memrealtime ticks (10 ns) of the loop.
// *instructions_per_wavefront counts matrix instructions (modes 0, 1, 3) or multiply-adds (mode 2).
extern "C" int pl_probe_alu_rate(int mode, int waves, unsigned long long* out_dev, int* sink_dev, void* stream, long long* instructions_per_wavefront) {
  if (!out_dev || !sink_dev || !instructions_per_wavefront || mode < 0 || mode > 3 || (waves != 4 && waves != 8)) return (int)hipErrorInvalidValue;
  *instructions_per_wavefront = (long long)kAluIters * (mode == 3 ? 4 : 8);
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e = hipSuccess;
  switch (mode) {
    case 0: e = LaunchAlu<0>(waves, out_dev, sink_dev, s); break;
    case 1: e = LaunchAlu<1>(waves, out_dev, sink_dev, s); break;
    case 2: e = LaunchAlu<2>(waves, out_dev, sink_dev, s); break;
    default: e = LaunchAlu<3>(waves, out_dev, sink_dev, s); break;
  }
  return (int)e;
}
