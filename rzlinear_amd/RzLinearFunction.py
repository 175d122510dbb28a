"""autograd.Function of the compressed linear layer (host side of the drop-in boundary).

Kept from the reference (python/rz_linear/RzLinearFunction.py:7-60): the module-global
``controls`` dict with its two ``triton_*`` keys, ``RzLinearFunction.apply(input, hashed_weight,
random_numbers, output_dim, chunk_size, init_factor)`` and a backward that hands autograd
``(input_grad, weight_grad, None, ...)``.
"""
import torch

from .impl.RzLinearBackward import (rz_linear_backward_input_grad_tl,
                                    rz_linear_backward_weight_bias_grad_tl,
                                    rz_linear_backward_weight_grad_tl)
from .impl.RzLinearForward import rz_linear_forward_bias_tl

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


def _launcher_kwargs(block_k, block_n):
    return dict(allow_tf32=controls['triton_allow_tf32'], allow_autotune=controls['triton_allow_autotune'],
                BLOCK_SIZE_K=block_k, BLOCK_SIZE_N=block_n)


def _hash_args(random_numbers):
    """R7..R0, the positional order of the launchers, from the 8-element CPU tensor."""
    assert random_numbers.numel() == 8
    return tuple(int(v) for v in reversed(random_numbers.tolist()))


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
        consts = _hash_args(random_numbers)
        tile = (int(controls['block_size_k'] if block_size_k is None else block_size_k),
                int(controls['block_size_n'] if block_size_n is None else block_size_n))
        M, K = input.shape
        H = hashed_weight.shape[0]
        output = rz_linear_forward_bias_tl(input, hashed_weight.data, None if bias is None else bias.data,
                                           init_factor, M, K, output_dim, H, *consts,
                                           **_launcher_kwargs(*tile))
        ctx.save_for_backward(input, hashed_weight, random_numbers)
        ctx.output_dim, ctx.chunk_size, ctx.init_factor = output_dim, chunk_size, init_factor
        ctx.tile = tile
        ctx.has_bias = bias is not None
        ctx.fuse_grad_accumulation = bool(fuse_grad_accumulation)
        return output

    @staticmethod
    def backward(ctx, grad):
        """One value per argument of forward (autograd drops trailing Nones that apply() was not
        given).  A gradient that autograd does not need is not computed — the reference always
        computes both."""
        input, hashed_weight, random_numbers = ctx.saved_tensors
        consts = _hash_args(random_numbers)
        M, K = input.shape
        N, H = ctx.output_dim, hashed_weight.shape[0]
        kwargs = _launcher_kwargs(*ctx.tile)
        need_input, need_weight = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_bias = ctx.has_bias and ctx.needs_input_grad[8]

        input_grad = weight_grad = bias_grad = None
        if need_input:      # enqueued first, like the reference's rz_linear_backward_tl
            input_grad = rz_linear_backward_input_grad_tl(grad, hashed_weight.data, ctx.init_factor,
                                                          M, K, N, H, *consts, **kwargs)
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
            launcher = rz_linear_backward_weight_bias_grad_tl if need_bias else rz_linear_backward_weight_grad_tl
            result = launcher(input, grad, ctx.init_factor, M, K, N, H, *consts, out=target, accumulate=accumulate,
                              **kwargs)
            bias_grad = result[1] if need_bias else None
        elif need_weight and need_bias:   # one pass over grad yields both
            weight_grad, bias_grad = rz_linear_backward_weight_bias_grad_tl(input, grad, ctx.init_factor,
                                                                            M, K, N, H, *consts, **kwargs)
        elif need_weight:
            weight_grad = rz_linear_backward_weight_grad_tl(input, grad, ctx.init_factor,
                                                            M, K, N, H, *consts, **kwargs)
        elif need_bias:
            bias_grad = grad.sum(dim=0)
        return input_grad, weight_grad, None, None, None, None, None, None, bias_grad, None
