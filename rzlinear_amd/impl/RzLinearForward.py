"""Forward launcher: Y = (X . W_hashed) * init_factor on the gfx950 HIP kernel."""
import torch

from .. import _lib


def rz_linear_forward_tl(input: torch.Tensor, hashed_weight: torch.Tensor, init_factor: float,
                         M: int, K: int, N: int, H: int,
                         R7: int, R6: int, R5: int, R4: int,
                         R3: int, R2: int, R1: int, R0: int,
                         allow_tf32: bool = True, allow_autotune: bool = True,
                         BLOCK_SIZE_M: int = 64, BLOCK_SIZE_N: int = 64, BLOCK_SIZE_K: int = 32,
                         GROUP_SIZE: int = 4) -> torch.Tensor:
    """Same signature and result as the reference launcher
    (python/rz_linear/impl/RzLinearForward.py:6-85).

    BLOCK_SIZE_K x BLOCK_SIZE_N is the hashed tile of W and decides the result; allow_tf32,
    allow_autotune, BLOCK_SIZE_M and GROUP_SIZE only steered the reference's scheduling and are
    accepted and ignored (fp32 always runs on true-fp32 MFMA).  Returns a new [M, N] tensor of
    input's dtype on input's device.
    """
    return rz_linear_forward_bias_tl(input, hashed_weight, None, init_factor, M, K, N, H,
                                     R7, R6, R5, R4, R3, R2, R1, R0, allow_tf32=allow_tf32,
                                     allow_autotune=allow_autotune, BLOCK_SIZE_M=BLOCK_SIZE_M,
                                     BLOCK_SIZE_N=BLOCK_SIZE_N, BLOCK_SIZE_K=BLOCK_SIZE_K,
                                     GROUP_SIZE=GROUP_SIZE)


def rz_linear_forward_bias_tl(input: torch.Tensor, hashed_weight: torch.Tensor, bias, init_factor: float,
                              M: int, K: int, N: int, H: int,
                              R7: int, R6: int, R5: int, R4: int,
                              R3: int, R2: int, R1: int, R0: int,
                              allow_tf32: bool = True, allow_autotune: bool = True,
                              BLOCK_SIZE_M: int = 64, BLOCK_SIZE_N: int = 64, BLOCK_SIZE_K: int = 32,
                              GROUP_SIZE: int = 4) -> torch.Tensor:
    """rz_linear_forward_tl with the module's bias (a [N] tensor or None) added inside the
    kernel's store, instead of by the separate ``x + self._bias`` of the reference module
    (python/rz_linear/RzLinear.py:93-94)."""
    assert (H > (BLOCK_SIZE_K * BLOCK_SIZE_N))
    return forward_hashed(input, hashed_weight, bias, init_factor, M, K, N, H,
                          _lib.hash_constants(R7, R6, R5, R4, R3, R2, R1, R0), BLOCK_SIZE_K, BLOCK_SIZE_N,
                          _lib.HASH_TWO_LEVEL)


def forward_hashed(input, hashed_weight, bias, init_factor, M, K, N, H, R, BK, BN, hash_levels):
    """One rz_forward_hashed call: R is the int32[8] constant array, hash_levels an rz_hash code."""
    stream = _lib.require_gpu(input, hashed_weight, *([bias] if bias is not None else []))
    if hashed_weight.dtype != input.dtype:
        raise TypeError("input is %s but hashed_weight is %s" % (input.dtype, hashed_weight.dtype))
    if bias is not None:
        if bias.dtype != input.dtype or bias.numel() != N:
            raise TypeError("bias must be a [%d] tensor of %s" % (N, input.dtype))
        bias = bias.contiguous()
    if M == 0:   # an empty batch: nothing to launch, as the reference returns its empty zeros((0, N))
        return torch.empty((0, N), device=input.device, dtype=input.dtype)
    x, ldx = _lib.rows(input)
    hw = hashed_weight.contiguous()
    output = torch.empty((M, N), device=input.device, dtype=input.dtype)
    lib = _lib.load()
    code = _lib.dtype_code(input)
    # skinny problems split the contraction and need a scratch buffer for the partial results
    tuning = _lib.current_tuning()
    need = _lib.host_query("rz_forward_hashed_workspace_bytes", M, K, N, H, BK, BN, code)
    ws = _lib.workspace(need, input.device)
    _lib.check(lib.rz_forward_hashed(
        x.data_ptr(), hw.data_ptr(), bias.data_ptr() if bias is not None else None, output.data_ptr(),
        ws.data_ptr() if need else None, need, M, K, N, H, BK, BN, R, hash_levels, float(init_factor),
        ldx, N, code, tuning, stream))
    return output
