"""GPU parity of the legacy-generation compatibility mode (hash_levels = 3, 16 x 16 tiles):
device hash bit-exact, the row the reference's notebook recorded, and forward / input-grad /
weight-grad against the CPU oracle evaluated with the same hash."""
import ctypes
import sys

import numpy as np
import pytest
import torch

from helpers import TOL, make_inputs, rel_err

pytestmark = pytest.mark.gpu

NOTEBOOK_ROW1 = sum((list(range(a, a + 16)) for a in (275, 433, 591, 597, 755, 168, 326, 484)), [])


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("cfg", [(128, 128, 1000, 16, 16), (99999, 16, 300, 16, 16), (40000, 500, 1000000, 16, 16),
                                 (4096, 4096, 16778, 64, 64), (64, 64, 256, 16, 16)],
                         ids=lambda c: "x".join(map(str, c)))
def test_device_legacy_offsets_bit_exact(oracle, cfg):
    from rzlinear_amd import _lib
    K, N, H, BK, BN = cfg
    _say("legacy offsets", cfg)
    lib = _lib.load()
    TK, TN = -(-K // BK), -(-N // BN)
    for seed in (1024, 3):
        R = oracle.legacy_constants(seed)
        out = torch.empty((TK, TN), dtype=torch.int32, device="cuda")
        _lib.check(lib.rz_tile_offsets_device(out.data_ptr(), K, N, H, BK, BN, (ctypes.c_int32 * 8)(*R), 3,
                                              torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().astype(np.int64), oracle.c_tile_offsets(K, N, H, BK, BN, R, 3))


def test_notebook_row_on_the_device(oracle):
    """hashed_weight = arange(1000), identity input, 128 x 128, seed 1024: row 1 of the output is
    the row the reference's notebook shows (verify.ipynb, cell 3)."""
    from rzlinear_amd.legacy import LegacyRzLinearFunction, legacy_random_numbers, legacy_weight
    _say("legacy notebook row")
    rn = legacy_random_numbers(1024)
    assert rn.dtype == torch.int64 and rn.shape == (51,)
    assert rn[:4].tolist() == [2038074743, 634329019, 1825252241, 871205357]
    hw = torch.arange(1000, dtype=torch.float32, device="cuda")
    out = LegacyRzLinearFunction.apply(hw, torch.eye(128, device="cuda"), rn, 128, 128, 1, True)
    torch.cuda.synchronize()
    assert out[1].cpu().long().tolist() == NOTEBOOK_ROW1
    W = legacy_weight(hw, rn, 128, 128)
    assert torch.equal(W, out)
    assert np.array_equal(W.cpu().numpy(), oracle.materialize(np.arange(1000), 128, 128, 16, 16,
                                                              oracle.legacy_constants(1024), 3))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", [(5, 400, 500, 100000), (256, 512, 256, 9000), (70, 100, 50, 256),
                                   (512, 1024, 1024, 65536)], ids=lambda s: "x".join(map(str, s)))
def test_legacy_forward_backward(oracle, shape, dtype):
    from rzlinear_amd.legacy import LegacyRzLinearFunction, legacy_random_numbers
    M, K, N, H = shape
    _say("legacy fwd/bwd", shape, dtype)
    seed = 11
    rn = legacy_random_numbers(seed)
    R = oracle.legacy_constants(seed)
    assert rn[:8].tolist() == R
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=21)
    x.requires_grad_(True)
    hw.requires_grad_(True)
    y = LegacyRzLinearFunction.apply(hw, x, rn, K, N, 1, True)
    y.backward(dy)
    torch.cuda.synchronize()
    assert rel_err(y.detach().float().cpu().numpy(), oracle.forward(x64, hw64, N, 16, 16, R, 1.0, 3)) <= TOL[dtype]
    assert rel_err(x.grad.float().cpu().numpy(), oracle.input_grad(dy64, hw64, K, 16, 16, R, 1.0, 3)) <= TOL[dtype]
    assert rel_err(hw.grad.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, 16, 16, R, 1.0, 3)) <= TOL[dtype]


def test_legacy_module(oracle):
    from rzlinear_amd.legacy import LegacyRzLinear
    _say("legacy module")
    hw = torch.nn.Parameter(((torch.rand(5000) * 2 - 1) / 10).cuda())
    m = LegacyRzLinear(96, 80, 1, hw, tiled=True, seed=5).cuda()
    with torch.no_grad():
        m.bias.copy_(torch.linspace(-1, 1, 80))
    x = torch.randn(2, 3, 96, device="cuda")
    y = m(x)
    torch.cuda.synchronize()
    assert y.shape == (2, 3, 80)
    R = oracle.legacy_constants(5)
    ref = oracle.forward(x.reshape(-1, 96).double().cpu().numpy(), hw.detach().double().cpu().numpy(), 80, 16, 16, R,
                         1.0, 3) + np.linspace(-1, 1, 80)
    assert rel_err(y.detach().reshape(-1, 80).cpu().numpy(), ref) <= TOL[torch.float32]
    y.sum().backward()
    assert hw.grad is not None and m.bias.grad is not None
    assert sorted(m.state_dict().keys()) == ["bias", "random_numbers", "weight"]
    with pytest.raises(NotImplementedError):
        LegacyRzLinear(96, 80, 1, hw, tiled=False)


def test_legacy_hash_through_the_fold_path_with_a_layer_plan(oracle, tuned, monkeypatch):
    """hash_levels = 3 with the tiles folded by the second kernel: the tile offsets come from a layer
    plan built with the legacy hash, or are hashed by the call itself — the same bits either way."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import weight_grad_hashed
    tuned(fold=1, window=-1)
    M, K, N, H = 96, 400, 336, 100000
    _say("legacy fold + plan")
    R = oracle.legacy_constants(5)
    Rc = (ctypes.c_int32 * 8)(*R)
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, torch.float32, seed=23)
    assert _lib.plan_query(2, M, K, N, H, 16, 16, _lib.RZ_F32)["mode"] == "fold"
    monkeypatch.setattr(_lib, "use_layer_plans", False)
    a = weight_grad_hashed(x, dy, 1.0, M, K, N, H, Rc, 16, 16, hash_levels=_lib.HASH_LEGACY)[0]
    monkeypatch.setattr(_lib, "use_layer_plans", True)
    b = weight_grad_hashed(x, dy, 1.0, M, K, N, H, Rc, 16, 16, hash_levels=_lib.HASH_LEGACY)[0]
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    assert rel_err(b.cpu().numpy(), oracle.weight_grad(x64, dy64, H, 16, 16, R, 1.0, 3)) <= TOL[torch.float32]
