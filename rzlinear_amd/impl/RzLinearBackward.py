"""Backward launchers: input-grad and weight-grad on the gfx950 HIP kernels."""
from typing import Tuple

import torch

from .. import _lib


def rz_linear_backward_tl(input: torch.Tensor, hashed_weight: torch.Tensor, output_grad: torch.Tensor,
                          init_factor: float,
                          M: int, K: int, N: int, H: int,
                          R7: int, R6: int, R5: int, R4: int,
                          R3: int, R2: int, R1: int, R0: int,
                          allow_tf32: bool = True, allow_autotune: bool = False,
                          BLOCK_SIZE_M: int = 64, BLOCK_SIZE_N: int = 64, BLOCK_SIZE_K: int = 32,
                          GROUP_SIZE: int = 4) -> Tuple[torch.Tensor, torch.Tensor]:
    """(input_grad, weight_grad), input-grad enqueued first as in the reference
    (python/rz_linear/impl/RzLinearBackward.py:7-20)."""
    input_grad = rz_linear_backward_input_grad_tl(
        output_grad, hashed_weight, init_factor, M, K, N, H, R7, R6, R5, R4, R3, R2, R1, R0,
        allow_tf32=allow_tf32, allow_autotune=allow_autotune, BLOCK_SIZE_M=BLOCK_SIZE_M,
        BLOCK_SIZE_N=BLOCK_SIZE_N, BLOCK_SIZE_K=BLOCK_SIZE_K, GROUP_SIZE=GROUP_SIZE)
    weight_grad = rz_linear_backward_weight_grad_tl(
        input, output_grad, init_factor, M, K, N, H, R7, R6, R5, R4, R3, R2, R1, R0,
        allow_tf32=allow_tf32, allow_autotune=allow_autotune, BLOCK_SIZE_M=BLOCK_SIZE_M,
        BLOCK_SIZE_N=BLOCK_SIZE_N, BLOCK_SIZE_K=BLOCK_SIZE_K, GROUP_SIZE=GROUP_SIZE)
    return input_grad, weight_grad


def weight_grad_hashed(input, output_grad, init_factor, M, K, N, H, R, BLOCK_SIZE_K, BLOCK_SIZE_N,
                       out=None, accumulate=False, with_bias_grad=False, hash_levels=_lib.HASH_TWO_LEVEL,
                       use_layer_plan=None):
    """One weight-grad call; returns (hashed_weight_grad, bias_grad or None).

    Where the library would work by windows of dHW or fold stored tiles into dHW (a hashed_weight
    too large for an image in LDS), the call goes through rz_weight_grad_planned with the layer's
    plan, which _lib.layer_plan builds once per (K, N, H, tile, constants) and keeps on the device;
    everything else, and use_layer_plan=False (default: _lib.use_layer_plans), goes through
    rz_weight_grad_hashed."""
    stream = _lib.require_gpu(input, output_grad)
    if input.dtype != output_grad.dtype:
        raise TypeError("input is %s but output_grad is %s" % (input.dtype, output_grad.dtype))
    lib = _lib.load()
    code = _lib.dtype_code(output_grad)
    flags = 0
    if out is None:
        if accumulate:
            raise ValueError("accumulate=True needs the buffer to add into (out=...)")
        out = torch.empty((H,), device=output_grad.device, dtype=output_grad.dtype)
    else:
        _lib.require_gpu(output_grad, out)
        if out.shape != (H,) or not out.is_contiguous():
            raise ValueError("out must be a contiguous tensor of %d elements" % H)
        if out.dtype == torch.float32:
            flags |= _lib.WG_DHW_F32
        elif out.dtype != output_grad.dtype:
            raise TypeError("out must be float32 or %s, got %s" % (output_grad.dtype, out.dtype))
        if accumulate:
            flags |= _lib.WG_ACCUMULATE
    if M == 0:   # an empty batch contributes a zero gradient (the reference returns its zeros(H))
        if not accumulate:
            out.zero_()
        return out, (torch.zeros((N,), device=output_grad.device, dtype=output_grad.dtype) if with_bias_grad else None)
    x, ldx = _lib.rows(input)
    dy, lddy = _lib.rows(output_grad)
    bias_grad = torch.empty((N,), device=output_grad.device, dtype=output_grad.dtype) if with_bias_grad else None
    tuning = _lib.current_tuning()
    need = _lib.host_query("rz_weight_grad_hashed_workspace_bytes", M, K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N, code,
                           flags, int(with_bias_grad))
    ws = _lib.workspace(need, output_grad.device)
    plan = None
    if use_layer_plan is None:
        use_layer_plan = _lib.use_layer_plans
    if use_layer_plan and _lib.plan_query(2, M, K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N, code, flags,
                                          with_bias_grad, planned=True)["mode"] in ("window", "fold"):
        plan = _lib.layer_plan(K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N, R, hash_levels, output_grad.device)
    if plan is not None:
        _lib.check(lib.rz_weight_grad_planned(
            x.data_ptr(), dy.data_ptr(), out.data_ptr(), bias_grad.data_ptr() if with_bias_grad else None,
            ws.data_ptr() if need else None, need, plan.data_ptr(), plan.numel() * 4, M, K, N, H, BLOCK_SIZE_K,
            BLOCK_SIZE_N, R, hash_levels, float(init_factor), ldx, lddy, code, flags, tuning, stream))
    else:
        _lib.check(lib.rz_weight_grad_hashed(
            x.data_ptr(), dy.data_ptr(), out.data_ptr(), bias_grad.data_ptr() if with_bias_grad else None,
            ws.data_ptr() if need else None, need, M, K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N, R, hash_levels,
            float(init_factor), ldx, lddy, code, flags, tuning, stream))
    return out, bias_grad


def rz_linear_backward_weight_grad_tl(input: torch.Tensor, output_grad: torch.Tensor, init_factor: float,
                                      M: int, K: int, N: int, H: int,
                                      R7: int, R6: int, R5: int, R4: int,
                                      R3: int, R2: int, R1: int, R0: int,
                                      allow_tf32: bool = True, allow_autotune: bool = True,
                                      BLOCK_SIZE_M: int = 64, BLOCK_SIZE_N: int = 64, BLOCK_SIZE_K: int = 32,
                                      GROUP_SIZE: int = 8, out: torch.Tensor = None,
                                      accumulate: bool = False) -> torch.Tensor:
    """hashed_weight_grad[H] = scatter_add over W tiles of (input^T . output_grad) * init_factor.

    Same signature as the reference launcher (python/rz_linear/impl/RzLinearBackward.py:23-97);
    the result has output_grad's dtype.  The tiles are reduced and scattered in fp32 whatever the
    dtype (the reference adds atomically in output_grad's dtype), then converted once.

    Beyond the reference: ``out`` (a [H] tensor of output_grad's dtype or float32) receives the
    result instead of a new tensor, and with ``accumulate=True`` the gradient is added to what
    ``out`` holds — for layers that share one hashed_weight and for fp32 master gradients.
    """
    R = _lib.hash_constants(R7, R6, R5, R4, R3, R2, R1, R0)
    return weight_grad_hashed(input, output_grad, init_factor, M, K, N, H, R, BLOCK_SIZE_K, BLOCK_SIZE_N,
                        out=out, accumulate=accumulate)[0]


def rz_linear_backward_weight_bias_grad_tl(input: torch.Tensor, output_grad: torch.Tensor, init_factor: float,
                                           M: int, K: int, N: int, H: int,
                                           R7: int, R6: int, R5: int, R4: int,
                                           R3: int, R2: int, R1: int, R0: int,
                                           allow_tf32: bool = True, allow_autotune: bool = True,
                                           BLOCK_SIZE_M: int = 64, BLOCK_SIZE_N: int = 64, BLOCK_SIZE_K: int = 32,
                                           GROUP_SIZE: int = 8, out: torch.Tensor = None,
                                           accumulate: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """(hashed_weight_grad[H], bias_grad[N]) from one pass over output_grad.

    bias_grad = output_grad.sum(0): the gradient of the bias that the reference module adds after
    the product (python/rz_linear/RzLinear.py:93-94) and leaves to autograd.  Here the
    weight-grad kernel sums the output_grad tiles it stages anyway.  No counterpart launcher in
    the reference; arguments as rz_linear_backward_weight_grad_tl.
    """
    R = _lib.hash_constants(R7, R6, R5, R4, R3, R2, R1, R0)
    return weight_grad_hashed(input, output_grad, init_factor, M, K, N, H, R, BLOCK_SIZE_K, BLOCK_SIZE_N,
                        out=out, accumulate=accumulate, with_bias_grad=True)


def rz_linear_backward_input_grad_tl(output_grad: torch.Tensor, hashed_weight: torch.Tensor, init_factor: float,
                                     M: int, K: int, N: int, H: int,
                                     R7: int, R6: int, R5: int, R4: int,
                                     R3: int, R2: int, R1: int, R0: int,
                                     allow_tf32: bool = True, allow_autotune: bool = True,
                                     BLOCK_SIZE_M: int = 64, BLOCK_SIZE_N: int = 64, BLOCK_SIZE_K: int = 32,
                                     GROUP_SIZE: int = 4) -> torch.Tensor:
    """input_grad[M, K] = (output_grad . W_hashed^T) * init_factor.

    Same signature as the reference launcher (python/rz_linear/impl/RzLinearBackward.py:374-449).
    """
    assert (H > (BLOCK_SIZE_K * BLOCK_SIZE_N))
    return input_grad_hashed(output_grad, hashed_weight, init_factor, M, K, N, H,
                             _lib.hash_constants(R7, R6, R5, R4, R3, R2, R1, R0), BLOCK_SIZE_K, BLOCK_SIZE_N,
                             _lib.HASH_TWO_LEVEL)


def input_grad_hashed(output_grad, hashed_weight, init_factor, M, K, N, H, R, BK, BN, hash_levels):
    """One rz_input_grad_hashed call: R is the int32[8] constant array, hash_levels an rz_hash code."""
    stream = _lib.require_gpu(output_grad, hashed_weight)
    if hashed_weight.dtype != output_grad.dtype:
        raise TypeError("output_grad is %s but hashed_weight is %s" % (output_grad.dtype, hashed_weight.dtype))
    if M == 0:
        return torch.empty((0, K), device=output_grad.device, dtype=output_grad.dtype)
    dy, lddy = _lib.rows(output_grad)
    hw = hashed_weight.contiguous()
    input_grad = torch.empty((M, K), device=output_grad.device, dtype=output_grad.dtype)
    lib = _lib.load()
    code = _lib.dtype_code(output_grad)
    tuning = _lib.current_tuning()
    need = _lib.host_query("rz_input_grad_hashed_workspace_bytes", M, K, N, H, BK, BN, code)
    ws = _lib.workspace(need, output_grad.device)
    _lib.check(lib.rz_input_grad_hashed(
        dy.data_ptr(), hw.data_ptr(), input_grad.data_ptr(), ws.data_ptr() if need else None, need,
        M, K, N, H, BK, BN, R, hash_levels, float(init_factor), lddy, K, code, tuning, stream))
    return input_grad
