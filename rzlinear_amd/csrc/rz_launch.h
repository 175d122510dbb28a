// Host-side launch of the contraction kernels; one translation unit per element type.
#pragma once

#include "rz_common.h"

namespace rz {

// Fills in the tiling fields of `p` and enqueues the kernel for `op` on `stream`.
hipError_t launch_gemm_f32(int op, GemmParams p, hipStream_t stream);
hipError_t launch_gemm_bf16(int op, GemmParams p, hipStream_t stream);
hipError_t launch_gemm_f16(int op, GemmParams p, hipStream_t stream);

}  // namespace rz
