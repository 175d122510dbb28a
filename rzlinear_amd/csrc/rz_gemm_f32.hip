// Instantiation of the contraction kernels for element type float.
#include "rz_gemm_inst.h"

namespace rz {
hipError_t launch_gemm_f32(int op, GemmParams p, const WeightGradPlan* plan, const SplitPlan* split,
                           const rz_tuning& tuning, hipStream_t stream) {
  return launch_gemm_t<float>(op, p, plan, split, tuning, stream);
}
hipError_t launch_window_f32(const WindowParams& p, int windows, hipStream_t stream) {
  return launch_window_t<float>(p, windows, stream);
}
}  // namespace rz
