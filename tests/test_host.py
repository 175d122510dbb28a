"""CPU checks of the host-side mirror of the reference interface (module, Function, launchers):
names, defaults, assertions, state_dict, and that nothing falls back to a CPU path."""
import inspect

import pytest
import torch

import rzlinear_amd
from rzlinear_amd import RzLinear, RzLinearFunction, controls
from rzlinear_amd.impl.RzLinearBackward import (rz_linear_backward_input_grad_tl, rz_linear_backward_tl,
                                                rz_linear_backward_weight_grad_tl)
from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
from rzlinear_amd.impl.RzLinearIdx import rz_linear_idx_tl

R1024 = [45007, 20011, 38363, 15263, 24507, 36489, 12234, 43027]


def test_module_construction_matches_reference_surface():
    m = RzLinear(input_dim=1024, output_dim=512)
    assert (m._input_dim, m._output_dim, m._chunk_size, m._seed) == (1024, 512, 1, 1024)
    assert m._compress_ratio == 0.0625 and m._init_factor == 1.0
    assert m._random_numbers.dtype == torch.int32 and m._random_numbers.device.type == "cpu"
    assert m._random_numbers.tolist() == R1024
    assert RzLinear.P == 45007 and RzLinear.R == 8
    H = int(1024 * 512 * 0.0625)
    assert m._hashed_weight.shape == (H,) and m._hashed_weight.dtype == torch.float32
    assert torch.equal(m._hashed_weight.data, torch.arange(H).float())     # arange init, as the reference
    assert list(m.state_dict().keys()) == ["_hashed_weight", "_bias"]
    assert m._bias.shape == (512,) and not m._bias.any()
    assert "RzLinear(mm=1024x512 bias=True seed=1024" in repr(m)
    assert (m._block_size_k, m._block_size_n) == (32, 64)                  # reference launcher defaults


def test_module_options():
    shared = torch.nn.Parameter(torch.zeros(5000, dtype=torch.bfloat16))
    a = RzLinear(64, 64, hashed_weight=shared, bias=False, seed=0, dtype=torch.bfloat16, init_factor=0.5,
                 block_size_k=64, block_size_n=64)
    b = RzLinear(64, 32, hashed_weight=shared, seed=0)
    assert a._hashed_weight is shared and b._hashed_weight is shared
    assert a._bias is False and list(a.state_dict().keys()) == ["_hashed_weight"]
    assert a._random_numbers.tolist() == [45007, 29440, 22221, 32190, 14791, 1316, 35275, 26448]
    # the draw reseeds torch's global generator, like the reference
    RzLinear(16, 16, seed=7)
    x = torch.rand(3)
    torch.manual_seed(7); torch.randint(0, 45007, (7,))
    assert torch.equal(x, torch.rand(3))


def test_assertions_of_the_reference():
    with pytest.raises(AssertionError):
        RzLinear(10**5, 16)
    with pytest.raises(AssertionError):
        RzLinear(16, 10**5)
    m = RzLinear(64, 64)
    with pytest.raises(AssertionError):
        m(torch.zeros(64))                                               # ndim < 2
    x = torch.zeros((4, 64)); hw = torch.zeros(2048)
    with pytest.raises(AssertionError):                                  # H <= BK*BN
        rz_linear_forward_tl(x, hw, 1.0, 4, 64, 64, 2048, *R1024[::-1], BLOCK_SIZE_K=32, BLOCK_SIZE_N=64)
    with pytest.raises(AssertionError):
        rz_linear_backward_input_grad_tl(x, hw, 1.0, 4, 64, 64, 2048, *R1024[::-1], BLOCK_SIZE_K=32,
                                         BLOCK_SIZE_N=64)
    with pytest.raises(AssertionError):                                  # 8 hash constants
        RzLinearFunction.apply(x, hw, torch.tensor(R1024[:4], dtype=torch.int32), 64, 1, 1.0)
    with pytest.raises(AssertionError):                                  # idx: K % BK, N % BN
        rz_linear_idx_tl(torch.zeros(70000), 100, 128, 70000, 1, 2, 3, 45007, 32, 32)


def test_launcher_signatures_are_the_reference_ones():
    def names(fn):
        return list(inspect.signature(fn).parameters)
    consts = ["R7", "R6", "R5", "R4", "R3", "R2", "R1", "R0"]
    tail = ["allow_tf32", "allow_autotune", "BLOCK_SIZE_M", "BLOCK_SIZE_N", "BLOCK_SIZE_K", "GROUP_SIZE"]
    dims = ["M", "K", "N", "H"]
    assert names(rz_linear_forward_tl) == ["input", "hashed_weight", "init_factor"] + dims + consts + tail
    assert names(rz_linear_backward_tl) == ["input", "hashed_weight", "output_grad", "init_factor"] + dims + consts + tail
    # the reference's arguments first, then this build's optional gradient-buffer arguments
    assert names(rz_linear_backward_weight_grad_tl) == (["input", "output_grad", "init_factor"] + dims + consts + tail +
                                                        ["out", "accumulate"])
    extra = inspect.signature(rz_linear_backward_weight_grad_tl).parameters
    assert extra["out"].default is None and extra["accumulate"].default is False
    assert names(rz_linear_backward_input_grad_tl) == ["output_grad", "hashed_weight", "init_factor"] + dims + consts + tail
    assert names(rz_linear_idx_tl) == ["hashed_weight", "K", "N", "H", "R3", "R2", "R1", "R0", "BLOCK_SIZE_K", "BLOCK_SIZE_N"]
    d = {k: v.default for k, v in inspect.signature(rz_linear_forward_tl).parameters.items()}
    assert (d["BLOCK_SIZE_M"], d["BLOCK_SIZE_N"], d["BLOCK_SIZE_K"], d["GROUP_SIZE"]) == (64, 64, 32, 4)
    assert inspect.signature(rz_linear_backward_weight_grad_tl).parameters["GROUP_SIZE"].default == 8
    assert controls["triton_allow_tf32"] is False and controls["triton_allow_autotune"] is False


def test_no_cpu_fallback():
    m = RzLinear(64, 64, compress_ratio=1.0)
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        m(torch.zeros((4, 64)))
    x = torch.zeros((4, 64)); hw = torch.zeros(8192)
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        rz_linear_backward_weight_grad_tl(x, x, 1.0, 4, 64, 64, 8192, *R1024[::-1])
    with pytest.raises(TypeError):
        from rzlinear_amd import _lib
        _lib.dtype_code(torch.zeros(1, dtype=torch.float64))


def test_product_never_imports_the_oracle():
    import os
    root = os.path.dirname(os.path.abspath(rzlinear_amd.__file__))
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), (f, "mentions the oracle")


def test_install_as_rz_linear():
    rzlinear_amd.install_as_rz_linear()
    import rz_linear
    from rz_linear import RzLinear as A, RzLinearFunction as B, controls as C
    from rz_linear.impl.RzLinearForward import rz_linear_forward_tl as f
    from rz_linear.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl, rz_linear_backward_input_grad_tl
    from rz_linear.impl.RzLinearIdx import rz_linear_idx_tl as g
    assert A is RzLinear and B is RzLinearFunction and C is controls and f is rz_linear_forward_tl
