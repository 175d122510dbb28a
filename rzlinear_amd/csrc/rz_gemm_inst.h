// Body shared by the per-dtype translation units: tile choice + launch.
#pragma once

#include <stdlib.h>

#include "rz_gemm.h"
#include "rz_launch.h"

namespace rz {

// Number of workgroups of the small tile that fills the 256 compute units a few times over.
static constexpr int kTargetWorkgroups = 1024;
static constexpr int kComputeUnits = 256;

template <typename T, int OP, int TI, int TJ, int WI, int WJ, int NSTAGE, bool FULL>
static hipError_t launch_one(GemmParams p, hipStream_t stream) {
  typedef GemmKernel<T, OP, TI, TJ, WI, WJ, NSTAGE, FULL> K;
  p.tiles_i = (p.I + TI - 1) / TI;
  p.tiles_j = (p.J + TJ - 1) / TJ;
  const long long tiles = (long long)p.tiles_i * p.tiles_j;
  if (tiles <= 0 || tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  int splits = 1;
  const int r_steps = (p.R + K::TR - 1) / K::TR;
  if (OP == kWeightGrad) {
    // split the reduction over M when there are too few W tiles to fill the chip
    const long long target = (TI >= 256) ? kComputeUnits : kTargetWorkgroups;
    long long want = (target + tiles - 1) / tiles;
    if (want > r_steps) want = r_steps;
    if (want < 1) want = 1;
    const int steps_per = (int)((r_steps + want - 1) / want);
    splits = (r_steps + steps_per - 1) / steps_per;
    p.r_chunk = steps_per * K::TR;
  } else {
    p.r_chunk = r_steps * K::TR;
  }
  auto kernel = rz_gemm_kernel<T, OP, TI, TJ, WI, WJ, NSTAGE, FULL>;
  constexpr size_t smem = sizeof(typename K::Smem);
  static_assert(smem <= 160 * 1024, "tile does not fit the 160 KB LDS of a compute unit");
  if (smem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  dim3 grid((unsigned)tiles, (unsigned)splits, 1), block(K::kThreads, 1, 1);
  hipLaunchKernelGGL(kernel, grid, block, smem, stream, p);
  return hipGetLastError();
}

// Large tile (256 x 256, one workgroup per compute unit, two LDS stages) when it still yields
// enough workgroups to occupy the chip; else the 128 x 128 tile with several workgroups per
// compute unit.  RZLINEAR_TILE=128|256 forces one of them (tuning aid).
static inline int pick_tile(const GemmParams& p) {
  static const int forced = []() {
    const char* e = getenv("RZLINEAR_TILE");
    return e ? atoi(e) : 0;
  }();
  if (forced == 128 || forced == 256) return forced;
  const long long big = (long long)((p.I + 255) / 256) * ((p.J + 255) / 256);
  return big >= kComputeUnits / 2 ? 256 : 128;
}

// FULL kernels carry no bounds checks: every tile and every R step must be complete.
template <typename T, int OP, int TILE, int NSTAGE>
static hipError_t launch_tile(GemmParams p, hipStream_t stream) {
  constexpr int TR = 128 / ElemTraits<T>::kBytes;
  // 256 x 256: eight wavefronts (two per SIMD) of 128 x 64; 128 x 128: four of 64 x 64
  constexpr int WJ = (TILE == 256) ? 4 : 2;
  const bool full = (p.I % TILE == 0) && (p.J % TILE == 0) && (p.R % TR == 0);
  if (full) return launch_one<T, OP, TILE, TILE, 2, WJ, NSTAGE, true>(p, stream);
  return launch_one<T, OP, TILE, TILE, 2, WJ, NSTAGE, false>(p, stream);
}

template <typename T>
static hipError_t launch_gemm_t(int op, GemmParams p, hipStream_t stream) {
  const int tile = pick_tile(p);
  if (tile == 256) {
    switch (op) {
      case kForward: return launch_tile<T, kForward, 256, 2>(p, stream);
      case kInputGrad: return launch_tile<T, kInputGrad, 256, 2>(p, stream);
      case kWeightGrad: return launch_tile<T, kWeightGrad, 256, 2>(p, stream);
      default: return hipErrorInvalidValue;
    }
  }
  switch (op) {
    case kForward: return launch_tile<T, kForward, 128, 1>(p, stream);
    case kInputGrad: return launch_tile<T, kInputGrad, 128, 1>(p, stream);
    case kWeightGrad: return launch_tile<T, kWeightGrad, 128, 1>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace rz
