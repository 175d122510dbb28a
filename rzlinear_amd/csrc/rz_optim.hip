// Fused optimiser steps over a parameter vector (the hashed_weight of one or several layers, or
// a bias): one pass over parameter, gradient and state instead of the handful of elementwise
// kernels of a generic optimiser.  The reference leaves the update to torch.optim; the update
// rules here are torch.optim.SGD's and torch.optim.Adam's / AdamW's.
#include "../../include/rzlinear.h"

#include <hip/hip_runtime.h>

#include "rz_common.h"

namespace rz {

struct SgdArgs {
  float lr, momentum, dampening, weight_decay, grad_scale;
  int nesterov, first_step;
};

struct AdamArgs {
  float lr, beta1, beta2, eps, weight_decay, grad_scale;
  float bias1, bias2_sqrt;   // 1 - beta1^t, sqrt(1 - beta2^t)
  int decoupled;
};

// The fp32 value of the parameter is its master copy when there is one (16-bit parameters whose
// small updates would otherwise be rounded away), else the parameter itself.
template <typename P, typename G>
__global__ __launch_bounds__(256) void sgd_step_kernel(P* __restrict__ param, const G* __restrict__ grad,
                                                       float* __restrict__ momentum_buf, float* __restrict__ master,
                                                       int64_t n, SgdArgs a) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float w = master != nullptr ? master[i] : ElemTraits<P>::to_float(param[i]);
    float g = ElemTraits<G>::to_float(grad[i]) * a.grad_scale;
    if (a.weight_decay != 0.f) g += a.weight_decay * w;
    if (a.momentum != 0.f) {
      const float b = a.first_step ? g : a.momentum * momentum_buf[i] + (1.f - a.dampening) * g;
      momentum_buf[i] = b;
      g = a.nesterov ? g + a.momentum * b : b;
    }
    w -= a.lr * g;
    if (master != nullptr) master[i] = w;
    param[i] = ElemTraits<P>::from_float(w);
  }
}

template <typename P, typename G>
__global__ __launch_bounds__(256) void adam_step_kernel(P* __restrict__ param, const G* __restrict__ grad,
                                                        float* __restrict__ exp_avg, float* __restrict__ exp_avg_sq,
                                                        float* __restrict__ master, int64_t n, AdamArgs a) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float w = master != nullptr ? master[i] : ElemTraits<P>::to_float(param[i]);
    float g = ElemTraits<G>::to_float(grad[i]) * a.grad_scale;
    if (a.weight_decay != 0.f) {
      if (a.decoupled) w *= 1.f - a.lr * a.weight_decay;
      else g += a.weight_decay * w;
    }
    const float m = a.beta1 * exp_avg[i] + (1.f - a.beta1) * g;
    const float v = a.beta2 * exp_avg_sq[i] + (1.f - a.beta2) * g * g;
    exp_avg[i] = m;
    exp_avg_sq[i] = v;
    const float denom = sqrtf(v) / a.bias2_sqrt + a.eps;
    w -= (a.lr / a.bias1) * (m / denom);
    if (master != nullptr) master[i] = w;
    param[i] = ElemTraits<P>::from_float(w);
  }
}

static inline unsigned blocks_for(int64_t n) {
  const int64_t b = (n + 255) / 256;
  return (unsigned)(b < 1 ? 1 : (b > 8192 ? 8192 : b));
}

// dispatch over (parameter type, gradient type: the parameter's own or fp32)
template <typename F>
static int with_types(int param_dtype, int grad_dtype, F&& f) {
  if (grad_dtype != param_dtype && grad_dtype != RZ_F32) return RZ_ERR_BAD_DTYPE;
  switch (param_dtype) {
    case RZ_F32: return f((float*)nullptr, (float*)nullptr);
    case RZ_BF16: return grad_dtype == RZ_F32 ? f((bf16_t*)nullptr, (float*)nullptr) : f((bf16_t*)nullptr, (bf16_t*)nullptr);
    case RZ_F16: return grad_dtype == RZ_F32 ? f((f16_t*)nullptr, (float*)nullptr) : f((f16_t*)nullptr, (f16_t*)nullptr);
    default: return RZ_ERR_BAD_DTYPE;
  }
}

}  // namespace rz

using namespace rz;

#define RZ_API __attribute__((visibility("default")))

extern "C" {

RZ_API int rz_sgd_step(void* param, const void* grad, float* momentum_buf, float* master, int64_t n,
                       int param_dtype, int grad_dtype, float lr, float momentum, float dampening,
                       float weight_decay, int nesterov, int first_step, float grad_scale, void* stream) {
  if (param == nullptr || grad == nullptr) return RZ_ERR_NULL_POINTER;
  if (momentum != 0.f && momentum_buf == nullptr) return RZ_ERR_NULL_POINTER;
  if (n < 0) return RZ_ERR_BAD_SHAPE;
  if (nesterov && (momentum <= 0.f || dampening != 0.f)) return RZ_ERR_BAD_ARGUMENT;   // as torch.optim.SGD
  if (n == 0) return RZ_OK;
  SgdArgs a = {lr, momentum, dampening, weight_decay, grad_scale, nesterov ? 1 : 0, first_step ? 1 : 0};
  return with_types(param_dtype, grad_dtype, [&](auto* p, auto* g) -> int {
    typedef typename std::remove_pointer<decltype(p)>::type P;
    typedef typename std::remove_pointer<decltype(g)>::type G;
    hipLaunchKernelGGL((sgd_step_kernel<P, G>), dim3(blocks_for(n)), dim3(256), 0, (hipStream_t)stream, (P*)param,
                       (const G*)grad, momentum_buf, master, n, a);
    return hipGetLastError() == hipSuccess ? RZ_OK : RZ_ERR_LAUNCH;
  });
}

RZ_API int rz_adam_step(void* param, const void* grad, float* exp_avg, float* exp_avg_sq, float* master, int64_t n,
                        int param_dtype, int grad_dtype, float lr, float beta1, float beta2, float eps,
                        float weight_decay, int decoupled, int step, float grad_scale, void* stream) {
  if (param == nullptr || grad == nullptr || exp_avg == nullptr || exp_avg_sq == nullptr) return RZ_ERR_NULL_POINTER;
  if (n < 0) return RZ_ERR_BAD_SHAPE;
  if (step < 1 || !(beta1 >= 0.f && beta1 < 1.f) || !(beta2 >= 0.f && beta2 < 1.f)) return RZ_ERR_BAD_ARGUMENT;
  if (n == 0) return RZ_OK;
  AdamArgs a = {lr, beta1, beta2, eps, weight_decay, grad_scale,
                (float)(1.0 - pow((double)beta1, (double)step)), (float)sqrt(1.0 - pow((double)beta2, (double)step)),
                decoupled ? 1 : 0};
  return with_types(param_dtype, grad_dtype, [&](auto* p, auto* g) -> int {
    typedef typename std::remove_pointer<decltype(p)>::type P;
    typedef typename std::remove_pointer<decltype(g)>::type G;
    hipLaunchKernelGGL((adam_step_kernel<P, G>), dim3(blocks_for(n)), dim3(256), 0, (hipStream_t)stream, (P*)param,
                       (const G*)grad, exp_avg, exp_avg_sq, master, n, a);
    return hipGetLastError() == hipSuccess ? RZ_OK : RZ_ERR_LAUNCH;
  });
}

}  // extern "C"
