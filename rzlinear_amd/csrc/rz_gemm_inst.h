// Body shared by the per-dtype translation units: tile choice + launch.
#pragma once

#include <atomic>

#include "rz_gemm.h"
#include "rz_launch.h"
#include "rz_window.h"

namespace rz {

template <typename T, int OP, int TI, int TJ, int WI, int WJ, int NSTAGE, bool FULL, bool COLSUM, bool CLAMP = false,
          int WK = 1>
static hipError_t launch_one(GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                             hipStream_t stream) {
  static std::atomic<uint64_t> lds_limit_raised{0};
  typedef GemmKernel<T, OP, TI, TJ, WI, WJ, NSTAGE, FULL, COLSUM, CLAMP, WK> K;
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
    // exactly one target: the tile-by-tile output, or an image (LDS mode: partial images) to scatter into
    if (plan->fold.use != (p.tiles_out != nullptr) || (p.tiles_out == nullptr) == (p.scatter == nullptr))
      return hipErrorInvalidValue;
    if (plan->fold.use && p.image_pitch > 0) return hipErrorInvalidValue;
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
    // a slice must begin on a step boundary: the offset table of a step assumes that the step
    // lies inside one hashed tile or covers whole ones
    if (p.r_chunk % K::TR != 0) return hipErrorInvalidValue;
    // (the kernel that finishes its own tiles holds the other slices' values in registers)
    if (p.finish != nullptr && splits > kFinishSlices) return hipErrorInvalidValue;
  } else {
    p.r_chunk = r_steps * K::TR;
    p.partial = nullptr;
    p.finish = nullptr;
  }
  auto kernel = rz_gemm_kernel<T, OP, TI, TJ, WI, WJ, NSTAGE, FULL, COLSUM, CLAMP, WK>;
  size_t smem = sizeof(typename K::Smem);
  static_assert(sizeof(typename K::Smem) <= 160 * 1024, "tile does not fit the 160 KB LDS of a compute unit");
  if (OP == kWeightGrad && p.image_pitch > 0) {
    // the dHW image and the scatter's offset table behind it may need more than the stages
    const size_t need = (size_t)p.image_pitch * sizeof(float) + (K::kOffEntries + K::kTurnEntries) * sizeof(int);
    if (need > smem) smem = need;
  }
  if (smem > 64 * 1024) {
    hipError_t e = raise_lds_limit(reinterpret_cast<const void*>(kernel), lds_limit_raised);
    if (e != hipSuccess) return e;
  }
  dim3 grid((unsigned)tiles, (unsigned)splits, 1), block(K::kThreads, 1, 1);
  hipLaunchKernelGGL(kernel, grid, block, smem, stream, p);
  return hipGetLastError();
}

// FULL kernels carry no bounds checks: every tile and every R step must be complete.  Ragged
// shapes: the directly staged forms (16-bit tiles of 128 and more, all two-stage fp32 forms) still
// stage directly, with edge pieces fetched from inside the operands (CLAMP); everything else takes
// the bounds-checked kernel.
template <typename T, int OP, int TILE, int WI, int WJ, int NSTAGE, bool COLSUM = false, int WK = 1, int TILE_J = TILE>
static hipError_t launch_tile(GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                              const KernelForm& form, hipStream_t stream) {
  // (the form was derived on the host from the same rules that select the instantiation here:
  //  refuse to launch if the two ever disagree about the step length)
  // A directly staged load addresses the hashed operand by a 32-bit byte offset from its first
  // element: an fp32 hashed_weight of 4 GB and more takes the bounds-checked kernel, whose loads
  // carry full pointers (the step is the same for both fp32 forms).
  const bool far = sizeof(T) == 4 && OP != kWeightGrad &&
                   ((unsigned long long)p.h.range + (unsigned long long)p.h.BK * (unsigned long long)p.h.BN) * sizeof(T) > 0xffffffffull;
  if (far) {
    if (form.step != GemmKernel<T, OP, TILE, TILE_J, WI, WJ, NSTAGE, false>::TR) return hipErrorInvalidValue;
    return launch_one<T, OP, TILE, TILE_J, WI, WJ, NSTAGE, false, COLSUM, false, WK>(p, plan, split, stream);
  }
  if (form.full) {
    if (form.step != GemmKernel<T, OP, TILE, TILE_J, WI, WJ, NSTAGE, true>::TR) return hipErrorInvalidValue;
    return launch_one<T, OP, TILE, TILE_J, WI, WJ, NSTAGE, true, COLSUM, false, WK>(p, plan, split, stream);
  }
  if constexpr (NSTAGE == 2 && (sizeof(T) == 4 || TILE >= 128)) {
    if (form.clamp) {
      if (form.step != GemmKernel<T, OP, TILE, TILE_J, WI, WJ, NSTAGE, false, false, true, WK>::TR) return hipErrorInvalidValue;
      return launch_one<T, OP, TILE, TILE_J, WI, WJ, NSTAGE, false, COLSUM, true, WK>(p, plan, split, stream);
    }
  }
  if (form.clamp || form.step != GemmKernel<T, OP, TILE, TILE_J, WI, WJ, NSTAGE, false>::TR) return hipErrorInvalidValue;
  return launch_one<T, OP, TILE, TILE_J, WI, WJ, NSTAGE, false, COLSUM, false, WK>(p, plan, split, stream);
}

template <typename T, int TILE, int WI, int WJ, int NSTAGE, int WK = 1>
static hipError_t launch_op(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                            const KernelForm& form, hipStream_t stream) {
  switch (op) {
    case kForward: return launch_tile<T, kForward, TILE, WI, WJ, NSTAGE, false, WK>(p, plan, split, form, stream);
    case kInputGrad: return launch_tile<T, kInputGrad, TILE, WI, WJ, NSTAGE, false, WK>(p, plan, split, form, stream);
    case kWeightGrad:
      if constexpr (WK == 1) {
        // with a column-sum target the kernel also produces the bias gradient's partial sums
        if (p.colsum != nullptr) return launch_tile<T, kWeightGrad, TILE, WI, WJ, NSTAGE, true>(p, plan, split, form, stream);
        return launch_tile<T, kWeightGrad, TILE, WI, WJ, NSTAGE>(p, plan, split, form, stream);
      }
      return hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
  }
}

// Tile shapes (all two LDS stages, software pipelined unless noted):
//   256: 256 x 256, eight wavefronts of 128 x 64, one workgroup per compute unit
//   128: 128 x 128, four wavefronts of 64 x 64 (up to two workgroups per compute unit) or
//        eight of 64 x 32 when there is about one workgroup per compute unit; tuning.stages = 1
//        selects a single-stage form that leans on several workgroups per compute unit
//        instead of a pipeline (tuning aid)
//    64:  64 x  64, four wavefronts of 32 x 32, for problems with few tiles; fp32 forward /
//        input-grad: eight, in two groups that share every R step between them
//    32:  32 x  64 (fp32 forward / input-grad whose rows would leave a 64-row tile at most half full): four wavefronts of 32 x 32 in two such groups
template <typename T>
static hipError_t launch_gemm_t(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                                const rz_tuning& tuning, hipStream_t stream) {
  const bool wg = op == kWeightGrad && plan != nullptr;
  const bool cut = !wg && split != nullptr && split->splits > 1;
  const int tile = wg ? plan->tile : (split != nullptr ? split->tile : pick_tile(p.I, p.J, (int)sizeof(T), tuning));
  const int chunk = wg ? plan->r_chunk : (cut ? split->r_chunk : p.R);
  const long long workgroups = wg ? plan->workgroups : tile_count(p.I, p.J, tile) * (cut ? split->splits : 1);
  const KernelForm form = kernel_form(op, p.I, p.J, p.R, chunk, tile, workgroups, (int)sizeof(T), tuning);
  switch (form.tile * 100 + form.waves * 10 + form.stages) {
    case 25682: return launch_op<T, 256, 2, 4, 2>(op, p, plan, split, form, stream);
    case 6442: return launch_op<T, 64, 2, 2, 2>(op, p, plan, split, form, stream);
    case 6482:   // fp32 forward / input-grad: two groups of four wavefronts share every R step
      if constexpr (sizeof(T) == 4) return launch_op<T, 64, 2, 2, 2, 2>(op, p, plan, split, form, stream);
      return hipErrorInvalidValue;
    case 3242:   // fp32 forward / input-grad, rows in 32s: 32 x 64, two groups of two wavefronts
      if constexpr (sizeof(T) == 4) {
        if (op == kForward) return launch_tile<T, kForward, 32, 1, 2, 2, false, 2, 64>(p, plan, split, form, stream);
        if (op == kInputGrad) return launch_tile<T, kInputGrad, 32, 1, 2, 2, false, 2, 64>(p, plan, split, form, stream);
      }
      return hipErrorInvalidValue;
    case 12841: return launch_op<T, 128, 2, 2, 1>(op, p, plan, split, form, stream);
    case 12882: return launch_op<T, 128, 2, 4, 2>(op, p, plan, split, form, stream);
    case 12842: return launch_op<T, 128, 2, 2, 2>(op, p, plan, split, form, stream);
    default: return hipErrorInvalidValue;
  }
}

template <typename T, int TBN, bool STAGED>
static hipError_t launch_window_form(const WindowParams& p, int windows, hipStream_t stream) {
  typedef WindowKernel<T, TBN, STAGED> K;
  static_assert(K::kFixedBytes + sizeof(float) * kWindowFloats <= 160 * 1024, "window does not fit the LDS");
  if (p.window < 4 || p.window > kWindowFloats || (p.window & 3) || windows < 1) return hipErrorInvalidValue;
  if ((long long)windows * p.window < p.H) return hipErrorInvalidValue;
  if (p.h.BN != TBN || !window_tile_supported(p.h.BK, p.h.BN)) return hipErrorInvalidValue;
  auto kernel = rz_window_kernel<T, TBN, STAGED>;
  const size_t smem = K::kFixedBytes + sizeof(float) * (size_t)p.window;
  static std::atomic<uint64_t> lds_limit_raised{0};
  if (smem > 64 * 1024) {
    hipError_t e = raise_lds_limit(reinterpret_cast<const void*>(kernel), lds_limit_raised);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)windows), dim3(K::kThreads), smem, stream, p);
  return hipGetLastError();
}

// Operands whose rows hold whole 16-byte pieces go through the staged form.
template <typename T, int TBN>
static hipError_t launch_window_one(const WindowParams& p, int windows, hipStream_t stream) {
  constexpr int kVec = 16 / (int)sizeof(T);
  // (the staged form keeps a lane's piece offsets, up to sixteen rows, in 32-bit registers)
  if (p.K % kVec == 0 && p.N % kVec == 0 && p.ldx < (1 << 26) && p.lddy < (1 << 26))
    return launch_window_form<T, TBN, true>(p, windows, stream);
  return launch_window_form<T, TBN, false>(p, windows, stream);
}

template <typename T>
static hipError_t launch_window_t(const WindowParams& p, int windows, hipStream_t stream) {
  if (p.h.BN == 64) return launch_window_one<T, 64>(p, windows, stream);
  if (p.h.BN == 32) return launch_window_one<T, 32>(p, windows, stream);
  if (p.h.BN == 128) return launch_window_one<T, 128>(p, windows, stream);
  return hipErrorInvalidValue;
}

}  // namespace rz
