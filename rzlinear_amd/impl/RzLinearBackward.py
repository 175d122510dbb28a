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


def rz_linear_backward_weight_grad_tl(input: torch.Tensor, output_grad: torch.Tensor, init_factor: float,
                                      M: int, K: int, N: int, H: int,
                                      R7: int, R6: int, R5: int, R4: int,
                                      R3: int, R2: int, R1: int, R0: int,
                                      allow_tf32: bool = True, allow_autotune: bool = True,
                                      BLOCK_SIZE_M: int = 64, BLOCK_SIZE_N: int = 64, BLOCK_SIZE_K: int = 32,
                                      GROUP_SIZE: int = 8) -> torch.Tensor:
    """hashed_weight_grad[H] = scatter_add over W tiles of (input^T . output_grad) * init_factor.

    Same signature as the reference launcher (python/rz_linear/impl/RzLinearBackward.py:23-97);
    the result has output_grad's dtype.  The tiles are reduced and scattered in fp32 whatever the
    dtype (the reference adds atomically in output_grad's dtype), then converted once.
    """
    stream = _lib.require_gpu(input, output_grad)
    if input.dtype != output_grad.dtype:
        raise TypeError("input is %s but output_grad is %s" % (input.dtype, output_grad.dtype))
    lib = _lib.load()
    x, ldx = _lib.rows(input)
    dy, lddy = _lib.rows(output_grad)
    code = _lib.dtype_code(output_grad)
    hashed_weight_grad = torch.empty((H,), device=output_grad.device, dtype=output_grad.dtype)
    need = lib.rz_weight_grad_workspace_bytes(M, K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N, code)
    workspace = torch.empty((max(need, 1),), device=output_grad.device, dtype=torch.uint8) if need else None
    _lib.check(lib.rz_weight_grad(
        x.data_ptr(), dy.data_ptr(), hashed_weight_grad.data_ptr(),
        workspace.data_ptr() if need else None, need, M, K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N,
        _lib.hash_constants(R7, R6, R5, R4, R3, R2, R1, R0), float(init_factor), ldx, lddy, code, stream))
    return hashed_weight_grad


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
    stream = _lib.require_gpu(output_grad, hashed_weight)
    if hashed_weight.dtype != output_grad.dtype:
        raise TypeError("output_grad is %s but hashed_weight is %s" % (output_grad.dtype, hashed_weight.dtype))
    dy, lddy = _lib.rows(output_grad)
    hw = hashed_weight.contiguous()
    input_grad = torch.empty((M, K), device=output_grad.device, dtype=output_grad.dtype)
    lib = _lib.load()
    code = _lib.dtype_code(output_grad)
    need = lib.rz_input_grad_workspace_bytes(M, K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N, code)
    ws = _lib.workspace(need, output_grad.device)
    _lib.check(lib.rz_input_grad_ws(
        dy.data_ptr(), hw.data_ptr(), input_grad.data_ptr(), ws.data_ptr() if need else None, need,
        M, K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N,
        _lib.hash_constants(R7, R6, R5, R4, R3, R2, R1, R0), float(init_factor), lddy, K, code, stream))
    return input_grad
