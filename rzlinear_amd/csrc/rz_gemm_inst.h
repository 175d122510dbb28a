// Body shared by the per-dtype translation units: tile choice + launch.
#pragma once

#include "rz_gemm.h"
#include "rz_launch.h"

namespace rz {

// Number of workgroups that fills the 256 compute units a few times over.
static constexpr int kTargetWorkgroups = 1024;

template <typename T, int OP, int TI, int TJ, int WI, int WJ>
static hipError_t launch_one(GemmParams p, hipStream_t stream) {
  typedef GemmKernel<T, OP, TI, TJ, WI, WJ> K;
  p.tiles_i = (p.I + TI - 1) / TI;
  p.tiles_j = (p.J + TJ - 1) / TJ;
  const long long tiles = (long long)p.tiles_i * p.tiles_j;
  if (tiles <= 0 || tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  int splits = 1;
  const int r_steps = (p.R + K::TR - 1) / K::TR;
  if (OP == kWeightGrad) {
    // split the reduction over M when there are too few W tiles to fill the chip
    long long want = (kTargetWorkgroups + tiles - 1) / tiles;
    if (want > r_steps) want = r_steps;
    if (want < 1) want = 1;
    const int steps_per = (int)((r_steps + want - 1) / want);
    splits = (r_steps + steps_per - 1) / steps_per;
    p.r_chunk = steps_per * K::TR;
  } else {
    p.r_chunk = r_steps * K::TR;
  }
  dim3 grid((unsigned)tiles, (unsigned)splits, 1), block(K::kThreads, 1, 1);
  hipLaunchKernelGGL((rz_gemm_kernel<T, OP, TI, TJ, WI, WJ>), grid, block, 0, stream, p);
  return hipGetLastError();
}

template <typename T>
static hipError_t launch_gemm_t(int op, GemmParams p, hipStream_t stream) {
  switch (op) {
    case kForward: return launch_one<T, kForward, 128, 128, 2, 2>(p, stream);
    case kInputGrad: return launch_one<T, kInputGrad, 128, 128, 2, 2>(p, stream);
    case kWeightGrad: return launch_one<T, kWeightGrad, 128, 128, 2, 2>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace rz
