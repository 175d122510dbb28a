// Body shared by the per-dtype translation units: tile choice + launch.
#pragma once

#include "rz_gemm.h"
#include "rz_launch.h"
#include "rz_window.h"

namespace rz {

template <typename T, int OP, int TI, int TJ, int WI, int WJ, int NSTAGE, bool FULL, bool COLSUM, bool CLAMP = false>
static hipError_t launch_one(GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                             hipStream_t stream) {
  typedef GemmKernel<T, OP, TI, TJ, WI, WJ, NSTAGE, FULL, COLSUM, CLAMP> K;
  p.tiles_i = (p.I + TI - 1) / TI;
  p.tiles_j = (p.J + TJ - 1) / TJ;
  const long long tiles = (long long)p.tiles_i * p.tiles_j;
  if (tiles <= 0 || tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  int splits = 1;
  const int r_steps = (p.R + K::TR - 1) / K::TR;
  if (OP == kWeightGrad) {
    if (plan == nullptr || plan->tile != TI) return hipErrorInvalidValue;
    splits = plan->splits;
    p.r_chunk = plan->r_chunk;
    p.image_pitch = plan->image_pitch;
    if ((size_t)p.image_pitch * sizeof(float) > kMaxImageBytes) return hipErrorInvalidValue;
    if (COLSUM) {
      if (p.colsum == nullptr || plan->colsum_pitch != p.tiles_j * TJ ||
          plan->colsum_rows != plan->splits * p.tiles_i)
        return hipErrorInvalidValue;
      p.colsum_pitch = plan->colsum_pitch;
    }
  } else if (split != nullptr && split->splits > 1) {
    if (split->tile != TI || p.partial == nullptr) return hipErrorInvalidValue;
    splits = split->splits;
    p.r_chunk = split->r_chunk;
  } else {
    p.r_chunk = r_steps * K::TR;
    p.partial = nullptr;
  }
  auto kernel = rz_gemm_kernel<T, OP, TI, TJ, WI, WJ, NSTAGE, FULL, COLSUM, CLAMP>;
  size_t smem = sizeof(typename K::Smem);
  static_assert(sizeof(typename K::Smem) <= 160 * 1024, "tile does not fit the 160 KB LDS of a compute unit");
  if (OP == kWeightGrad && p.image_pitch > 0) {
    // the dHW image and the scatter's offset table behind it may need more than the stages
    const size_t need = (size_t)p.image_pitch * sizeof(float) + K::kOffEntries * sizeof(int);
    if (need > smem) smem = need;
  }
  if (smem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  dim3 grid((unsigned)tiles, (unsigned)splits, 1), block(K::kThreads, 1, 1);
  hipLaunchKernelGGL(kernel, grid, block, smem, stream, p);
  return hipGetLastError();
}

// FULL kernels carry no bounds checks: every tile and every R step must be complete.
template <typename T, int OP, int TILE, int WI, int WJ, int NSTAGE, bool COLSUM = false>
static hipError_t launch_tile(GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                              hipStream_t stream) {
  // (the unchecked kernel's R step; every slice of a split contraction must be whole steps too)
  constexpr int TR = GemmKernel<T, OP, TILE, TILE, WI, WJ, NSTAGE, true>::TR;
  const int chunk = (OP == kWeightGrad) ? (plan != nullptr ? plan->r_chunk : p.R)
                                        : (split != nullptr && split->splits > 1 ? split->r_chunk : p.R);
  const bool full = (p.I % TILE == 0) && (p.J % TILE == 0) && (p.R % TR == 0) && (chunk % TR == 0);
  if (full) return launch_one<T, OP, TILE, TILE, WI, WJ, NSTAGE, true, COLSUM>(p, plan, split, stream);
  // Ragged shapes: 16-bit tiles can still be staged directly, with edge pieces fetched from
  // inside the operands.  A plain operand's 16-byte pieces must not straddle the end of its
  // rows: forward / input-grad need R, weight-grad needs I and J, to be multiples of the piece.
  if constexpr (sizeof(T) == 2 && NSTAGE == 2 && TILE >= 128) {
    constexpr int VEC = ElemTraits<T>::kVec;
    const bool pieces_ok = OP == kWeightGrad ? (p.I % VEC == 0 && p.J % VEC == 0 && p.I >= VEC && p.J >= VEC)
                                             : (p.R % VEC == 0 && p.R >= VEC);
    if (pieces_ok && getenv("RZLINEAR_NO_CLAMP") == nullptr)
      return launch_one<T, OP, TILE, TILE, WI, WJ, NSTAGE, false, COLSUM, true>(p, plan, split, stream);
  }
  return launch_one<T, OP, TILE, TILE, WI, WJ, NSTAGE, false, COLSUM>(p, plan, split, stream);
}

template <typename T, int TILE, int WI, int WJ, int NSTAGE>
static hipError_t launch_op(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                            hipStream_t stream) {
  switch (op) {
    case kForward: return launch_tile<T, kForward, TILE, WI, WJ, NSTAGE>(p, plan, split, stream);
    case kInputGrad: return launch_tile<T, kInputGrad, TILE, WI, WJ, NSTAGE>(p, plan, split, stream);
    case kWeightGrad:
      // with a column-sum target the kernel also produces the bias gradient's partial sums
      if (p.colsum != nullptr) return launch_tile<T, kWeightGrad, TILE, WI, WJ, NSTAGE, true>(p, plan, split, stream);
      return launch_tile<T, kWeightGrad, TILE, WI, WJ, NSTAGE>(p, plan, split, stream);
    default: return hipErrorInvalidValue;
  }
}

// Tile shapes (all two LDS stages, software pipelined unless noted):
//   256: 256 x 256, eight wavefronts of 128 x 64, one workgroup per compute unit
//   128: 128 x 128, four wavefronts of 64 x 64 (up to two workgroups per compute unit) or
//        eight of 64 x 32 when there is about one workgroup per compute unit
//    64:  64 x  64, four wavefronts of 32 x 32, for problems with few tiles
// RZLINEAR_STAGES=1 selects a single-stage 128 x 128 form that leans on several workgroups
// per compute unit instead of a pipeline (tuning aid).
template <typename T>
static hipError_t launch_gemm_t(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                                hipStream_t stream) {
  const int tile = (op == kWeightGrad && plan != nullptr) ? plan->tile
                   : (split != nullptr ? split->tile : pick_tile(p.I, p.J, (int)sizeof(T)));
  const char* stages_env = getenv("RZLINEAR_STAGES");
  const bool one_stage = stages_env != nullptr && atoi(stages_env) == 1;
  switch (tile) {
    case 256: return launch_op<T, 256, 2, 4, 2>(op, p, plan, split, stream);
    case 64: return launch_op<T, 64, 2, 2, 2>(op, p, plan, split, stream);
    case 128:
      if (one_stage) return launch_op<T, 128, 2, 2, 1>(op, p, plan, split, stream);
      // with about one workgroup per compute unit, eight wavefronts (two per SIMD, 64 x 32
      // each) hide latency better than four of 64 x 64; with more workgroups resident the
      // four-wavefront form does less LDS traffic per flop
      if (tile_count(p.I, p.J, 128) * (op == kWeightGrad && plan != nullptr ? plan->splits : 1) <=
          kComputeUnits * 3 / 2)
        return launch_op<T, 128, 2, 4, 2>(op, p, plan, split, stream);
      return launch_op<T, 128, 2, 2, 2>(op, p, plan, split, stream);
    default: return hipErrorInvalidValue;
  }
}

template <typename T, int TBK, int TBN>
static hipError_t launch_window_one(const WindowParams& p, int windows, hipStream_t stream) {
  typedef WindowKernel<T, TBK, TBN> K;
  static_assert(K::kFixedBytes + sizeof(float) * kWindowFloats <= 160 * 1024, "window does not fit the LDS");
  if (p.window < 4 || p.window > kWindowFloats || (p.window & 3) || windows < 1) return hipErrorInvalidValue;
  if ((long long)windows * p.window < p.H) return hipErrorInvalidValue;
  auto kernel = rz_window_kernel<T, TBK, TBN>;
  const size_t smem = K::kFixedBytes + sizeof(float) * (size_t)p.window;
  if (smem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)windows), dim3(K::kThreads), smem, stream, p);
  return hipGetLastError();
}

template <typename T>
static hipError_t launch_window_t(const WindowParams& p, int windows, hipStream_t stream) {
  if (p.h.BK == 64 && p.h.BN == 64) return launch_window_one<T, 64, 64>(p, windows, stream);
  if (p.h.BK == 32 && p.h.BN == 64) return launch_window_one<T, 32, 64>(p, windows, stream);
  return hipErrorInvalidValue;
}

}  // namespace rz
