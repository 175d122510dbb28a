"""nn.Module front-end of the compressed linear layer (host side of the drop-in boundary)."""
import torch
from torch.nn.parameter import Parameter

from .RzLinearFunction import RzLinearFunction


class RzLinear(torch.nn.Module):
    '''
        A linear layer whose [input_dim, output_dim] weight is read, tile by tile, out of a much
        smaller 1-D hashed_weight parameter (ROBE-Z).  Constructor arguments, attribute names,
        parameter names and the hash constants derived from `seed` are those of the reference
        (python/rz_linear/RzLinear.py:7-97).

        P (int): the prime of the hash, R (int): number of hash constants.
    '''
    P = 45007
    R = 8

    def __init__(self, input_dim: int, output_dim: int, chunk_size: int = 1,
                 hashed_weight: Parameter = None, tiled=True, seed: int = 1024, bias: bool = True,
                 dtype: torch.dtype = torch.float32, compress_ratio: float = 0.0625,
                 init_factor: float = 1.0, block_size_k: int = 32, block_size_n: int = 64) -> None:
        '''
            Args:
                input_dim (int): features of each input sample (K)
                output_dim (int): features of each output sample (N)
                chunk_size (int): stored and carried, unused (as in the reference)
                hashed_weight (Parameter): reuse this compressed weight instead of creating one
                tiled: accepted and ignored (as in the reference)
                seed (int): seed of the hash constants
                bias (bool): add a learnable bias
                dtype: dtype of the parameters
                compress_ratio (float): H = int(input_dim * output_dim * compress_ratio)
                init_factor (float): scale applied to the product
                block_size_k, block_size_n (int): hashed tile of W, powers of two in [16, 256];
                    the defaults are the reference's launcher defaults.  The same tile is used by
                    forward, input-grad and weight-grad, which is what makes them see one W.
        '''
        super(RzLinear, self).__init__()

        # the hash is evaluated in 32-bit integers
        assert (input_dim < 10**5 and output_dim < 10**5)

        self._input_dim = input_dim
        self._output_dim = output_dim
        self._compress_ratio = compress_ratio
        self._chunk_size = chunk_size
        self._hashed_weight = hashed_weight
        self._bias = bias
        self._seed = seed
        self._init_factor = init_factor
        self._block_size_k = block_size_k
        self._block_size_n = block_size_n

        # hash constants always live on the CPU and are not part of state_dict
        self._random_numbers = self._generate_random_numbers(seed)

        if hashed_weight is None:
            self._hashed_weight = Parameter(
                torch.arange(int(input_dim * output_dim * compress_ratio)).type(dtype))
        else:
            self._hashed_weight = hashed_weight

        if bias:
            self._bias = Parameter(torch.zeros(self._output_dim, dtype=dtype))

    def __repr__(self):
        return 'RzLinear(mm={}x{} bias={} seed={} hashed_weight_size={}, init_factor={} hashed_weight_id={})'.format(
            self._input_dim, self._output_dim, (self._bias is not None), self._seed,
            self._hashed_weight.size(), self._init_factor, self._hashed_weight.data_ptr())

    def _generate_random_numbers(self, seed: int):
        # Same draw as the reference (RzLinear.py:68-74), including that it reseeds torch's
        # global CPU generator: [P, 7 x randint(0, P)] as int32.
        torch.manual_seed(seed)
        x = torch.randint(0, RzLinear.P, (RzLinear.R - 1,)).type(torch.int32).requires_grad_(False)
        x = torch.cat([torch.tensor([RzLinear.P], dtype=torch.int32), x])
        return x.requires_grad_(False).cpu()

    def forward(self, x) -> torch.Tensor:
        '''
            Args:
                x (Tensor): (*, input_dim), at least 2-D

            Returns:
                output (Tensor): (*, output_dim)
        '''
        assert (len(x.shape) >= 2)
        dim_gt_2 = x.dim() > 2
        if (dim_gt_2):
            shape = x.shape
            x = x.reshape(-1, shape[-1]).contiguous()
        # the bias is added inside the forward kernel's store (one rounding, no extra pass)
        bias = self._bias if isinstance(self._bias, torch.Tensor) else None
        x = RzLinearFunction.apply(
            x, self._hashed_weight, self._random_numbers, self._output_dim, self._chunk_size,
            self._init_factor, self._block_size_k, self._block_size_n, bias)
        if (dim_gt_2):
            x = x.view(*shape[:-1], x.shape[-1])
        return x
