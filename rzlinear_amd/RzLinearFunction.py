"""autograd.Function of the compressed linear layer (host side of the drop-in boundary).

Kept from the reference (python/rz_linear/RzLinearFunction.py:7-60): the module-global
``controls`` dict with its two ``triton_*`` keys, ``RzLinearFunction.apply(input, hashed_weight,
random_numbers, output_dim, chunk_size, init_factor)`` and a backward that hands autograd
``(input_grad, weight_grad, None, ...)``.
"""
import torch

from . import _lib
from .impl.RzLinearBackward import input_grad_hashed, weight_grad_hashed
from .impl.RzLinearForward import forward_hashed

# Code written against the reference sets these two switches; they are accepted and have no
# effect here (no autotuner; fp32 is true fp32).  block_size_k / block_size_n give the hashed
# tile used when apply() is called without tile arguments — the reference launchers' defaults
# (RzLinearForward.py:11).
controls = {
    'triton_allow_tf32': False,
    'triton_allow_autotune': False,
    'block_size_k': 32,
    'block_size_n': 64,
}


def _hash_constants(random_numbers):
    """The int32[8] array of the C ABI (index = subscript) from the 8-element CPU tensor."""
    assert random_numbers.numel() == 8
    r = random_numbers.tolist()
    return _lib.hash_constants(r[7], r[6], r[5], r[4], r[3], r[2], r[1], r[0])


class RzLinearFunction(torch.autograd.Function):
    """output = (input @ W_hashed) * init_factor (+ bias).

    forward(input[M, K], hashed_weight[H], random_numbers[8] (CPU), output_dim, chunk_size,
            init_factor, block_size_k=None, block_size_n=None, bias=None,
            fuse_grad_accumulation=False) -> [M, output_dim]

    The first six arguments are the reference's; chunk_size is carried and unused, as there.
    The optional ones select the hashed tile (default: ``controls``), fuse the layer's bias into
    the forward kernel, and make backward add the weight gradient into the parameter's own
    gradient buffer instead of returning it (see RzLinear).
    """

    @staticmethod
    def forward(ctx, input, hashed_weight, random_numbers, output_dim, chunk_size, init_factor,
                block_size_k=None, block_size_n=None, bias=None, fuse_grad_accumulation=False):
        R = _hash_constants(random_numbers)
        tile = (int(controls['block_size_k'] if block_size_k is None else block_size_k),
                int(controls['block_size_n'] if block_size_n is None else block_size_n))
        M, K = input.shape
        H = hashed_weight.shape[0]
        assert (H > (tile[0] * tile[1]))   # (the launchers' assertion, impl/RzLinearForward.py:28 in the reference)
        output = forward_hashed(input, hashed_weight.data, None if bias is None else bias.data, init_factor,
                                M, K, output_dim, H, R, tile[0], tile[1], _lib.HASH_TWO_LEVEL)
        ctx.save_for_backward(input, hashed_weight, random_numbers)
        ctx.output_dim, ctx.chunk_size, ctx.init_factor = output_dim, chunk_size, init_factor
        ctx.tile = tile
        ctx.hash_constants = R   # (the ctypes array: backward need not convert the tensor again)
        ctx.has_bias = bias is not None
        ctx.fuse_grad_accumulation = bool(fuse_grad_accumulation)
        return output

    @staticmethod
    def backward(ctx, grad):
        """One value per argument of forward (autograd drops trailing Nones that apply() was not
        given).  A gradient that autograd does not need is not computed — the reference always
        computes both."""
        input, hashed_weight, _ = ctx.saved_tensors
        R = ctx.hash_constants
        M, K = input.shape
        N, H = ctx.output_dim, hashed_weight.shape[0]
        BK, BN = ctx.tile
        need_input, need_weight = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_bias = ctx.has_bias and ctx.needs_input_grad[8]

        input_grad = weight_grad = bias_grad = None
        if need_input:      # enqueued first, like the reference's rz_linear_backward_tl
            input_grad = input_grad_hashed(grad, hashed_weight.data, ctx.init_factor, M, K, N, H, R, BK, BN,
                                           _lib.HASH_TWO_LEVEL)
        if need_weight and ctx.fuse_grad_accumulation:
            # Add into the parameter's gradient buffer inside the kernels.  The first layer to
            # reach a parameter without a gradient overwrites a fresh buffer (no zero-fill), the
            # others accumulate; autograd gets no weight gradient and so adds nothing itself.
            target = getattr(hashed_weight, 'main_grad', None)
            accumulate = True
            if target is None:
                if hashed_weight.grad is None:
                    hashed_weight.grad = torch.empty_like(hashed_weight)
                    accumulate = False
                target = hashed_weight.grad
            _, bias_grad = weight_grad_hashed(input, grad, ctx.init_factor, M, K, N, H, R, BK, BN, out=target,
                                              accumulate=accumulate, with_bias_grad=need_bias)
        elif need_weight:   # (with a bias: one pass over grad yields both gradients)
            weight_grad, bias_grad = weight_grad_hashed(input, grad, ctx.init_factor, M, K, N, H, R, BK, BN,
                                                        with_bias_grad=need_bias)
        elif need_bias:
            bias_grad = grad.sum(dim=0)
        return input_grad, weight_grad, None, None, None, None, None, None, bias_grad, None
