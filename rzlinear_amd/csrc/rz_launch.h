// Host-side launch of the contraction kernels; one translation unit per element type.
#pragma once

#include "rz_common.h"

#include <stdlib.h>

namespace rz {

static constexpr int kComputeUnits = 256;
// Number of workgroups of the small tile that fills the compute units a few times over.
static constexpr int kTargetWorkgroups = 1024;

// Large tile (256 x 256, one workgroup of eight wavefronts per compute unit, two LDS stages)
// when it still yields enough workgroups to occupy the chip; else the 128 x 128 tile with
// several workgroups per compute unit.  RZLINEAR_TILE=128|256 forces one of them (tuning aid).
static inline int pick_tile(int I, int J) {
  static const int forced = []() {
    const char* e = getenv("RZLINEAR_TILE");
    return e ? atoi(e) : 0;
  }();
  if (forced == 128 || forced == 256) return forced;
  const long long big = (long long)((I + 255) / 256) * ((J + 255) / 256);
  return big >= kComputeUnits / 2 ? 256 : 128;
}

// How the weight-grad contraction C[K,N] = X^T.dY over M is cut into workgroups, and how the
// finished tiles reach dHW.
struct WeightGradPlan {
  int tile;          // C tile edge (128 or 256)
  int splits;        // slices of the reduction over M (blockIdx.y)
  int r_chunk;       // rows of M per slice, a multiple of the R step
  long long workgroups;
  int image_pitch;   // > 0: every workgroup first sums its tiles into an fp32 image of dHW held
                     // in LDS and stores it as one partial image; a second kernel adds the
                     // partial images up.  0: tiles go to dHW by global atomics.
  size_t workspace_bytes;
};

// LDS bytes that the weight-grad kernel's operand stages occupy (and its dHW image may reuse).
static inline size_t weight_grad_stage_bytes(int tile, int elem_bytes) {
  const int TR = 128 / elem_bytes;
  const size_t pitch = (elem_bytes == 2) ? (size_t)tile + 32 : (size_t)tile + 4;
  const size_t one = ((pitch * TR + 7) / 8) * 8 * elem_bytes;   // one operand, one stage
  return one * 2 * (tile == 256 ? 2 : 1);
}

static inline WeightGradPlan plan_weight_grad(int M, int K, int N, int H, int elem_bytes) {
  WeightGradPlan pl;
  pl.tile = pick_tile(K, N);
  const int TR = 128 / elem_bytes;
  const long long tiles = (long long)((K + pl.tile - 1) / pl.tile) * ((N + pl.tile - 1) / pl.tile);
  const int r_steps = (M + TR - 1) / TR;
  // split the reduction over M when there are too few W tiles to fill the chip
  const long long target = (pl.tile >= 256) ? kComputeUnits : kTargetWorkgroups;
  long long want = (target + tiles - 1) / tiles;
  if (want > r_steps) want = r_steps;
  if (want < 1) want = 1;
  const int steps_per = (int)((r_steps + want - 1) / want);
  pl.splits = (r_steps + steps_per - 1) / steps_per;
  pl.r_chunk = steps_per * TR;
  pl.workgroups = tiles * pl.splits;
  const int pitch = (H + 3) & ~3;
  static const bool no_image = getenv("RZLINEAR_NO_LDS_IMAGE") != nullptr;   // tuning aid
  const bool fits = (size_t)pitch * sizeof(float) <= weight_grad_stage_bytes(pl.tile, elem_bytes);
  pl.image_pitch = (fits && !no_image) ? pitch : 0;
  size_t ws = 0;
  if (pl.image_pitch > 0) ws = (size_t)pl.workgroups * pl.image_pitch * sizeof(float);
  else if (elem_bytes == 2) ws = (size_t)H * sizeof(float);   // fp32 image for the atomics
  pl.workspace_bytes = ws;
  return pl;
}

// Fills in the tiling fields of `p` and enqueues the kernel for `op` on `stream`; weight-grad
// takes its plan (tile, split of M, scatter mode) from `plan`, the others ignore it.
hipError_t launch_gemm_f32(int op, GemmParams p, const WeightGradPlan* plan, hipStream_t stream);
hipError_t launch_gemm_bf16(int op, GemmParams p, const WeightGradPlan* plan, hipStream_t stream);
hipError_t launch_gemm_f16(int op, GemmParams p, const WeightGradPlan* plan, hipStream_t stream);

}  // namespace rz
