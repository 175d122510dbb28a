// Measurement aid: what this GPU sustains on the MFMA work of one 256 x 256 C tile per compute unit
// when nothing else is in the way.  The dense peak of the data sheet is clock x MFMA width at the
// boost clock; under matrix load with real (non-constant) operands the clock is lower, and by how
// much is a property of the board that only a measurement gives.  The kernel below has the shape of
// the contraction kernels' inner loop — eight wavefronts per compute unit, 32 MFMA 32x32x16 per
// wavefront and step on eight accumulator blocks — and nothing else: its operands come out of
// registers (mode 0) or, like the real fragments, out of LDS with one barrier per step (mode 1).
// It reads no global memory inside the loop and writes one float per thread at the end.
#include "../../include/rzlinear.h"

#include <hip/hip_runtime.h>

#include "rz_common.h"

namespace rz {

template <typename T> struct ProbeMfma;
template <> struct ProbeMfma<bf16_t> {
  static __device__ __forceinline__ f32x16_t run(u32x4_t a, u32x4_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <> struct ProbeMfma<f16_t> {
  static __device__ __forceinline__ f32x16_t run(u32x4_t a, u32x4_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

static constexpr int kProbeThreads = 512;
static constexpr int kProbeLdsBytes = 65536;   // one stage of a 256 x 256 tile: 32 KB of each operand

// operands: 64 KB of 16-bit values (the caller's choice: random values draw the power real data draws)
// ticks[2 * workgroup] = shader clocks, [2 * workgroup + 1] = ticks of the constant 100 MHz clock, both
// over the loop of the workgroup's first wavefront
template <typename T, int MODE>
__global__ __launch_bounds__(kProbeThreads) void mfma_probe_kernel(const uint32_t* __restrict__ operands, float* __restrict__ out,
                                                                 unsigned long long* __restrict__ ticks, int steps) {
  extern __shared__ __attribute__((aligned(16))) unsigned char probe_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  f32x16_t acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[i][e] = 0.f;
  u32x4_t fa[4], fb[2];
#pragma unroll
  for (int i = 0; i < 4; i++) fa[i] = *reinterpret_cast<const u32x4_t*>(operands + (i * 64 + lane) * 4);
#pragma unroll
  for (int i = 0; i < 2; i++) fb[i] = *reinterpret_cast<const u32x4_t*>(operands + ((4 + i) * 64 + lane) * 4);
  if (MODE == 1) {
    for (int i = threadIdx.x; i < kProbeLdsBytes / 4; i += kProbeThreads) reinterpret_cast<uint32_t*>(probe_lds)[i] = operands[i];
    __syncthreads();
  }
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int s = 0; s < steps; s++) {
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      if (MODE == 1) {
        // six fragments of 1 KB per wavefront and sub-step, as a 128 x 64 wavefront tile reads them
        const unsigned char* base = probe_lds + ks * 4096 + lane * 16;
#pragma unroll
        for (int i = 0; i < 4; i++) fa[i] = *reinterpret_cast<const u32x4_t*>(base + (((wave & 1) * 4 + i) * 16384 + (s & 3) * 1024) % 32768);
#pragma unroll
        for (int i = 0; i < 2; i++) fb[i] = *reinterpret_cast<const u32x4_t*>(base + 32768 + (((wave >> 1) * 2 + i) * 16384 + (s & 3) * 1024) % 32768);
      }
#pragma unroll
      for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) acc[a * 2 + b] = ProbeMfma<T>::run(fa[a], fb[b], acc[a * 2 + b]);
    }
    if (MODE == 1) __syncthreads();
  }
  const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int e = 0; e < 16; e++) sum += acc[i][e];
  out[blockIdx.x * kProbeThreads + threadIdx.x] = sum;
  if (threadIdx.x == 0) {
    ticks[2 * blockIdx.x] = c1 - c0;
    ticks[2 * blockIdx.x + 1] = r1 - r0;
  }
}

}  // namespace rz

extern "C" __attribute__((visibility("default"))) int rz_mfma_probe(const void* operands, void* out, void* ticks, int workgroups,
                                                                    int steps, int mode, int dtype, void* stream) {
  using namespace rz;
  if (operands == nullptr || out == nullptr || ticks == nullptr) return RZ_ERR_NULL_POINTER;
  if (workgroups < 1 || workgroups > 65536 || steps < 1 || (mode != 0 && mode != 1)) return RZ_ERR_BAD_ARGUMENT;
  if (dtype != RZ_BF16 && dtype != RZ_F16) return RZ_ERR_BAD_DTYPE;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)workgroups), block(kProbeThreads);
  const uint32_t* src = static_cast<const uint32_t*>(operands);
  float* o = static_cast<float*>(out);
  unsigned long long* t = static_cast<unsigned long long*>(ticks);
  const size_t lds = mode == 1 ? kProbeLdsBytes : 0;
  if (dtype == RZ_BF16 && mode == 0) hipLaunchKernelGGL((mfma_probe_kernel<bf16_t, 0>), grid, block, lds, s, src, o, t, steps);
  else if (dtype == RZ_BF16) hipLaunchKernelGGL((mfma_probe_kernel<bf16_t, 1>), grid, block, lds, s, src, o, t, steps);
  else if (mode == 0) hipLaunchKernelGGL((mfma_probe_kernel<f16_t, 0>), grid, block, lds, s, src, o, t, steps);
  else hipLaunchKernelGGL((mfma_probe_kernel<f16_t, 1>), grid, block, lds, s, src, o, t, steps);
  return hipGetLastError() == hipSuccess ? RZ_OK : RZ_ERR_LAUNCH;
}
