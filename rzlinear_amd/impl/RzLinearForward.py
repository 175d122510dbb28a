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
    assert (H > (BLOCK_SIZE_K * BLOCK_SIZE_N))
    stream = _lib.require_gpu(input, hashed_weight)
    if hashed_weight.dtype != input.dtype:
        raise TypeError("input is %s but hashed_weight is %s" % (input.dtype, hashed_weight.dtype))
    x, ldx = _lib.rows(input)
    hw = hashed_weight.contiguous()
    output = torch.empty((M, N), device=input.device, dtype=input.dtype)
    _lib.check(_lib.load().rz_forward(
        x.data_ptr(), hw.data_ptr(), output.data_ptr(), M, K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N,
        _lib.hash_constants(R7, R6, R5, R4, R3, R2, R1, R0), float(init_factor), ldx, N,
        _lib.dtype_code(input), stream))
    return output
