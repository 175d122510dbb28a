"""Materialise the virtual weight W[K, N] from hashed_weight (test and inspection helper)."""
import torch

from .. import _lib


def rz_linear_idx_tl(hashed_weight: torch.Tensor,
                     K: int, N: int, H: int,
                     R3: int, R2: int, R1: int, R0: int,
                     BLOCK_SIZE_K: int = 32, BLOCK_SIZE_N: int = 32) -> torch.Tensor:
    """Same signature, hash and checks as the reference (python/rz_linear/impl/RzLinearIdx.py:6-45):
    the ONE-level hash ((tk*R3 + tn*R2 + R1) % R0) % (H - BK*BN), which is not the hash the
    forward/backward kernels use.  See rz_linear_weight_tl for the W those kernels see."""
    assert (H > (BLOCK_SIZE_K * BLOCK_SIZE_N))
    assert (K % BLOCK_SIZE_K == 0)
    assert (N % BLOCK_SIZE_N == 0)
    return _materialize(hashed_weight, K, N, H, (0, 0, 0, 0, R3, R2, R1, R0), BLOCK_SIZE_K, BLOCK_SIZE_N, 1)


def rz_linear_weight_tl(hashed_weight: torch.Tensor,
                        K: int, N: int, H: int,
                        R7: int, R6: int, R5: int, R4: int,
                        R3: int, R2: int, R1: int, R0: int,
                        BLOCK_SIZE_K: int = 32, BLOCK_SIZE_N: int = 64) -> torch.Tensor:
    """W[K, N] under the two-level hash of the forward/backward kernels
    (python/rz_linear/impl/RzLinearForward.py:316); K and N need not divide by the tile."""
    assert (H > (BLOCK_SIZE_K * BLOCK_SIZE_N))
    return _materialize(hashed_weight, K, N, H, (R7, R6, R5, R4, R3, R2, R1, R0), BLOCK_SIZE_K, BLOCK_SIZE_N, 2)


def _materialize(hashed_weight, K, N, H, consts, BK, BN, levels):
    stream = _lib.require_gpu(hashed_weight)
    hw = hashed_weight.contiguous()
    weight = torch.empty((K, N), device=hashed_weight.device, dtype=hashed_weight.dtype)
    _lib.check(_lib.load().rz_materialize(
        hw.data_ptr(), weight.data_ptr(), K, N, H, BK, BN, _lib.hash_constants(*consts), levels, N,
        _lib.dtype_code(hashed_weight), stream))
    return weight
