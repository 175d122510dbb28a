"""Compatibility front-end for hashed weights laid out by the LEGACY generation of RzLinear.

The legacy generation (/RzLinear.py, /rz_linear_kernel.cu of the reference) maps W[i, j] to
``hashed_weight[((i//16 * R3 + j//16 * R2 + R1) % R0) % (H - 255) + (i % 16) * 16 + j % 16]``
in 64-bit integers, with R0 = 2038074743 and R1.. drawn from numpy's RandomState(seed)
(/RzLinear.py:70-75, /rz_linear_kernel.cu:34-36,:56-64).  That is the tile scheme of the current
kernels with 16 x 16 tiles and another offset function, so the same HIP kernels run it
(``hash_levels = 3`` of the C ABI).  Only the tiled mode exists here; the legacy per-element
"chunk" mode (tiled=False) is not built.

Same call shapes as the legacy module: ``LegacyRzLinear(input_dim, output_dim, chunk_size,
hashed_weight, tiled=True, seed=1024)`` and ``LegacyRzLinearFunction.apply(hashed_weights,
input_v, random_numbers, input_dim, output_dim, chunk_size, tiled)``.
"""
import ctypes

import numpy as np
import torch
from torch import nn

from . import _lib
from .impl.RzLinearBackward import input_grad_hashed, weight_grad_hashed
from .impl.RzLinearForward import forward_hashed

LEGACY_PRIME = 2038074743
LEGACY_TILE = 16


def legacy_random_numbers(seed: int) -> torch.Tensor:
    """The 51 int64 numbers of the legacy module: the prime, then 50 odd numbers below it
    (/RzLinear.py:70-75).  Only the first four enter the tiled hash."""
    x = np.random.RandomState(seed).randint(0, LEGACY_PRIME, (50,))
    x = x + 1 * (x % 2 == 0)
    return torch.from_numpy(np.concatenate([np.array([LEGACY_PRIME]), x]).astype(np.int64))


def _constants(random_numbers):
    r = [int(v) for v in random_numbers[:4].tolist()]
    return (ctypes.c_int32 * 8)(r[0], r[1], r[2], r[3], 0, 0, 0, 0)


def _require_tiled(tiled):
    if not tiled:
        raise NotImplementedError("only the tiled layout of the legacy generation is supported")


def legacy_weight(hashed_weight: torch.Tensor, random_numbers, input_dim: int, output_dim: int) -> torch.Tensor:
    """W[input_dim, output_dim] as the legacy tiled kernels see it (inspection helper)."""
    stream = _lib.require_gpu(hashed_weight)
    hw = hashed_weight.contiguous()
    weight = torch.empty((input_dim, output_dim), device=hw.device, dtype=hw.dtype)
    _lib.check(_lib.load().rz_materialize(
        hw.data_ptr(), weight.data_ptr(), input_dim, output_dim, hw.shape[0], LEGACY_TILE, LEGACY_TILE,
        _constants(random_numbers), _lib.HASH_LEGACY, output_dim, _lib.dtype_code(hw), stream))
    return weight


class LegacyRzLinearFunction(torch.autograd.Function):
    """output = input_v @ W_legacy; backward returns (weight_grad, input_grad, None, ...), the
    argument order of the legacy Function (/RzLinear.py:12-37)."""

    @staticmethod
    def forward(ctx, hashed_weights, input_v, random_numbers, input_dim, output_dim, chunk_size, tiled):
        _require_tiled(tiled)
        M = input_v.shape[0]
        output = forward_hashed(input_v, hashed_weights.data, None, 1.0, M, input_dim, output_dim,
                                hashed_weights.shape[0], _constants(random_numbers), LEGACY_TILE, LEGACY_TILE,
                                _lib.HASH_LEGACY)
        ctx.save_for_backward(hashed_weights, input_v, random_numbers)
        ctx.dims = (input_dim, output_dim)
        return output

    @staticmethod
    def backward(ctx, grad):
        hashed_weights, input_v, random_numbers = ctx.saved_tensors
        K, N = ctx.dims
        M, H = input_v.shape[0], hashed_weights.shape[0]
        R = _constants(random_numbers)
        in_grad = wt_grad = None
        if ctx.needs_input_grad[1]:
            in_grad = input_grad_hashed(grad, hashed_weights.data, 1.0, M, K, N, H, R, LEGACY_TILE, LEGACY_TILE,
                                        _lib.HASH_LEGACY)
        if ctx.needs_input_grad[0]:
            wt_grad = weight_grad_hashed(input_v, grad, 1.0, M, K, N, H, R, LEGACY_TILE, LEGACY_TILE,
                                         hash_levels=_lib.HASH_LEGACY)[0]
        return wt_grad, in_grad, None, None, None, None, None


class LegacyRzLinear(nn.Module):
    """The legacy module's interface (/RzLinear.py:50-94): attributes ``weight`` (the shared
    hashed weight), ``bias``, ``random_numbers``; y = x @ W_legacy + bias."""

    def __init__(self, input_dim: int, output_dim: int, chunk_size: int, hashed_weight: torch.Tensor,
                 tiled=True, seed=1024) -> None:
        super().__init__()
        _require_tiled(tiled)
        self.input_dim, self.output_dim, self.chunk_size = input_dim, output_dim, chunk_size
        self.weight = hashed_weight
        self.memory_size = hashed_weight.size(0)
        self.tiled = tiled
        # kept as a Parameter for state_dict compatibility; the kernels take the host copy
        self.random_numbers = nn.Parameter(legacy_random_numbers(seed), requires_grad=False)
        self._host_random_numbers = legacy_random_numbers(seed)
        self.bias = nn.Parameter(torch.zeros(output_dim, dtype=hashed_weight.dtype))

    def forward(self, input_v: torch.Tensor) -> torch.Tensor:
        x = input_v if input_v.dim() <= 2 else input_v.reshape(-1, input_v.shape[-1])
        out = LegacyRzLinearFunction.apply(self.weight, x, self._host_random_numbers, self.input_dim,
                                           self.output_dim, self.chunk_size, self.tiled)
        out = out + self.bias
        return out if input_v.dim() <= 2 else out.view(*input_v.shape[:-1], out.shape[-1])
