// Instantiation of the contraction kernels for element type bf16_t.
#include "rz_gemm_inst.h"

namespace rz {
hipError_t launch_gemm_bf16(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                            const rz_tuning& tuning, hipStream_t stream) {
  return launch_gemm_t<bf16_t>(op, p, plan, split, tuning, stream);
}
hipError_t launch_window_bf16(const WindowParams& p, int windows, hipStream_t stream) {
  return launch_window_t<bf16_t>(p, windows, stream);
}
}  // namespace rz
