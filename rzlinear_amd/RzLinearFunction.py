"""autograd.Function of the compressed linear layer (host side of the drop-in boundary)."""
import torch

from .impl.RzLinearForward import rz_linear_forward_bias_tl
from .impl.RzLinearBackward import (rz_linear_backward_input_grad_tl,
                                    rz_linear_backward_weight_grad_tl)

# Module-global switches, same keys as the reference (python/rz_linear/RzLinearFunction.py:7-9).
# The two triton_* keys are kept so that code which sets them keeps working; they have no
# effect here (no autotuner, fp32 is true fp32).  block_size_k / block_size_n are the hashed
# tile used when RzLinearFunction.apply is called without explicit tile arguments; the
# defaults are the reference launchers' defaults (RzLinearForward.py:11).
controls = {}
controls['triton_allow_tf32'] = False
controls['triton_allow_autotune'] = False
controls['block_size_k'] = 32
controls['block_size_n'] = 64


class RzLinearFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input: torch.Tensor, hashed_weight: torch.Tensor,
                random_numbers: torch.Tensor, output_dim, chunk_size, init_factor,
                block_size_k=None, block_size_n=None, bias=None) -> torch.Tensor:
        '''
            Same six leading arguments and result as the reference
            (python/rz_linear/RzLinearFunction.py:13-43).

            Args:
                input (Tensor): (M, input_dim)
                hashed_weight (Tensor): (H), the compressed weight
                random_numbers (Tensor): (8) hash constants R0..R7 on the CPU
                output_dim (int): N
                chunk_size (int): carried, unused (as in the reference)
                init_factor (float): scale applied to every result
                block_size_k, block_size_n (int, optional): hashed tile; default controls[...]
                bias (Tensor, optional): (output_dim), added inside the kernel's store

            Returns:
                output (Tensor): (M, output_dim)
        '''
        assert (random_numbers.numel() == 8)
        R = [int(v) for v in random_numbers.tolist()]
        BK = int(block_size_k if block_size_k is not None else controls['block_size_k'])
        BN = int(block_size_n if block_size_n is not None else controls['block_size_n'])
        M, K, N, H = input.shape[0], input.shape[1], output_dim, hashed_weight.shape[0]
        output = rz_linear_forward_bias_tl(input, hashed_weight.data, None if bias is None else bias.data,
                                           init_factor, M, K, N, H,
                                           R[7], R[6], R[5], R[4], R[3], R[2], R[1], R[0],
                                           allow_tf32=controls['triton_allow_tf32'],
                                           allow_autotune=controls['triton_allow_autotune'],
                                           BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        ctx.save_for_backward(input, hashed_weight, random_numbers)
        ctx.output_dim = output_dim
        ctx.chunk_size = chunk_size
        ctx.init_factor = init_factor
        ctx.block_sizes = (BK, BN)
        ctx.has_bias = bias is not None
        return output

    @staticmethod
    def backward(ctx, grad):
        '''(input_grad, weight_grad, None, ...) — python/rz_linear/RzLinearFunction.py:45-60.
        A gradient that autograd does not need is skipped (the reference always computes both).'''
        input, hashed_weight, random_numbers = ctx.saved_tensors
        assert (random_numbers.numel() == 8)
        R = [int(v) for v in random_numbers.tolist()]
        BK, BN = ctx.block_sizes
        init_factor = ctx.init_factor
        M, K, N, H = input.shape[0], input.shape[1], ctx.output_dim, hashed_weight.shape[0]
        input_grad = weight_grad = None
        if ctx.needs_input_grad[0]:
            input_grad = rz_linear_backward_input_grad_tl(
                grad, hashed_weight.data, init_factor, M, K, N, H,
                R[7], R[6], R[5], R[4], R[3], R[2], R[1], R[0],
                allow_tf32=controls['triton_allow_tf32'], allow_autotune=controls['triton_allow_autotune'],
                BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        if ctx.needs_input_grad[1]:
            weight_grad = rz_linear_backward_weight_grad_tl(
                input, grad, init_factor, M, K, N, H,
                R[7], R[6], R[5], R[4], R[3], R[2], R[1], R[0],
                allow_tf32=controls['triton_allow_tf32'], allow_autotune=controls['triton_allow_autotune'],
                BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        bias_grad = None
        if ctx.has_bias and ctx.needs_input_grad[8]:
            bias_grad = grad.sum(dim=0)
        # autograd takes one value per argument that apply() was given (6 to 9 of them)
        return (input_grad, weight_grad, None, None, None, None, None, None, bias_grad)
