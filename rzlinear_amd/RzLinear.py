"""nn.Module front-end of the ROBE-Z compressed linear layer (host side of the drop-in boundary).

Interface contract kept from the reference module (python/rz_linear/RzLinear.py:7-97):
constructor arguments and defaults, the class constants ``P`` and ``R``, the private attribute
names that callers and tests read (``_input_dim``, ``_output_dim``, ``_compress_ratio``,
``_chunk_size``, ``_hashed_weight``, ``_bias``, ``_seed``, ``_init_factor``,
``_random_numbers``), the parameter names in ``state_dict`` and the way the hash constants are
drawn from ``seed``.
"""
import torch
from torch import nn

from .RzLinearFunction import RzLinearFunction

_INT32_SAFE_DIM = 10 ** 5   # the tile hash is evaluated in 32-bit integers


def draw_hash_constants(seed: int, prime: int, count: int) -> torch.Tensor:
    """[prime, count-1 integers in [0, prime)] as a CPU int32 tensor.

    Same draw as the reference (RzLinear.py:68-74): it reseeds torch's global CPU generator with
    ``seed`` and takes ``count - 1`` values of ``torch.randint``, so a given seed yields the same
    constants — and leaves the generator in the same state — as the reference module does.
    """
    torch.manual_seed(seed)
    tail = torch.randint(0, prime, (count - 1,)).to(torch.int32)
    head = torch.tensor([prime], dtype=torch.int32)
    return torch.cat((head, tail)).cpu().requires_grad_(False)


class RzLinear(nn.Module):
    """y = (x @ W) * init_factor + bias, where tile (tk, tn) of the virtual W[input_dim, output_dim]
    is a block_size_k x block_size_n slice of the 1-D ``hashed_weight`` at a hashed offset.

    Args:
        input_dim, output_dim: K and N of the virtual weight (both below 1e5).
        chunk_size: carried through to the autograd function, unused (as in the reference).
        hashed_weight: share this Parameter instead of creating one (several layers may).
        tiled: accepted and ignored (as in the reference).
        seed: seed of the eight hash constants.
        bias: learnable bias of size output_dim.
        dtype: dtype of the parameters (float32, bfloat16 or float16).
        compress_ratio: a new hashed_weight gets int(input_dim * output_dim * compress_ratio)
            elements, initialised to 0, 1, 2, ... like the reference's.
        init_factor: scale applied to the product.
        block_size_k, block_size_n: hashed tile, powers of two in [16, 256]; one tile for
            forward, input-grad and weight-grad, which is what makes the three see the same W.
            The defaults are the reference launchers' defaults.
        fuse_grad_accumulation: backward adds this layer's weight gradient straight into the
            parameter's gradient buffer (``hashed_weight.main_grad`` if the parameter carries such
            a [H] tensor — float32 master gradients — else ``hashed_weight.grad``) inside the
            weight-grad kernels, and hands autograd no weight gradient.  Layers that share one
            hashed_weight (python/rz_linear/RzLinear.py:54-58) then cost no extra pass over H per
            layer and no zero-fill.  Like every fused accumulation it bypasses gradient hooks on
            the parameter and higher-order differentiation through it.
    """

    P = 45007   # prime of the hash
    R = 8       # number of hash constants

    def __init__(self, input_dim: int, output_dim: int, chunk_size: int = 1,
                 hashed_weight: nn.Parameter = None, tiled=True, seed: int = 1024, bias: bool = True,
                 dtype: torch.dtype = torch.float32, compress_ratio: float = 0.0625,
                 init_factor: float = 1.0, block_size_k: int = 32, block_size_n: int = 64,
                 fuse_grad_accumulation: bool = False) -> None:
        super().__init__()
        assert input_dim < _INT32_SAFE_DIM and output_dim < _INT32_SAFE_DIM

        # geometry and hashing
        self._input_dim, self._output_dim = input_dim, output_dim
        self._block_size_k, self._block_size_n = block_size_k, block_size_n
        self._fuse_grad_accumulation = fuse_grad_accumulation
        self._chunk_size = chunk_size
        self._seed = seed
        self._random_numbers = self._generate_random_numbers(seed)   # plain attribute: stays on the CPU

        # numerics
        self._compress_ratio = compress_ratio
        self._init_factor = init_factor

        # parameters; `_bias` stays the bool False when there is no bias, as in the reference
        if hashed_weight is None:
            size = int(input_dim * output_dim * compress_ratio)
            hashed_weight = nn.Parameter(torch.arange(size).type(dtype))
        self._hashed_weight = hashed_weight
        self._bias = nn.Parameter(torch.zeros(output_dim, dtype=dtype)) if bias else False

    def _generate_random_numbers(self, seed: int) -> torch.Tensor:
        return draw_hash_constants(seed, RzLinear.P, RzLinear.R)

    def __repr__(self) -> str:
        return ('RzLinear(mm={}x{} bias={} seed={} hashed_weight_size={}, init_factor={} hashed_weight_id={})'
                .format(self._input_dim, self._output_dim, self._bias is not None, self._seed,
                        self._hashed_weight.size(), self._init_factor, self._hashed_weight.data_ptr()))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x: (*, input_dim) with at least two dimensions -> (*, output_dim)."""
        assert x.dim() >= 2
        lead = x.shape[:-1]
        rows = x if x.dim() == 2 else x.reshape(-1, x.shape[-1]).contiguous()
        # the bias is added inside the forward kernel's store (one rounding, no extra pass)
        bias = self._bias if isinstance(self._bias, torch.Tensor) else None
        out = RzLinearFunction.apply(rows, self._hashed_weight, self._random_numbers, self._output_dim,
                                     self._chunk_size, self._init_factor, self._block_size_k,
                                     self._block_size_n, bias, self._fuse_grad_accumulation)
        return out if x.dim() == 2 else out.view(*lead, out.shape[-1])
