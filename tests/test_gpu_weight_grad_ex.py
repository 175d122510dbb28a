"""GPU parity of rz_weight_grad_ex: bias gradient from the same pass, accumulation into an
existing buffer, fp32 gradient buffers for 16-bit operands.  Checked against the CPU oracle's
weight-grad and against the column sums of dY in float64."""
import ctypes
import sys

import numpy as np
import pytest
import torch

from helpers import SEED_CONSTANTS, TOL, make_inputs, rargs, rel_err

pytestmark = pytest.mark.gpu

R1024 = SEED_CONSTANTS[1024]

# (M, K, N, H, BK, BN)
CASES = [
    (512, 512, 512, 9000, 64, 64),       # complete tiles, LDS image
    (300, 200, 330, 9000, 32, 64),       # ragged
    (256, 256, 512, 70000, 64, 64),      # H too large for the LDS image: tiles stored and folded (fold = -1: global atomics)
    (130, 70, 90, 2000, 16, 16),         # 16-wide tiles
    (4100, 192, 160, 30000, 64, 64),     # long M: the reduction is cut into slices
    (40, 1500, 140, 9000, 64, 64),       # more tile rows than R steps: some workgroups never sum
]
ENVS = [{}, {"tile": 64}, {"tile": 128}, {"tile": 256}, {"tile": 128, "stages": 1}, {"lds_image": -1},
        {"lds_image": -1, "fold": -1}]   # rz_tuning overrides
_env_id = lambda e: "-".join("%s=%s" % (k, v) for k, v in e.items()) or "auto"
_dt_id = lambda d: str(d).split(".")[-1]
_shape_id = lambda s: "x".join(map(str, s))


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=_dt_id)
@pytest.mark.parametrize("env", ENVS, ids=_env_id)
@pytest.mark.parametrize("shape", CASES, ids=_shape_id)
def test_bias_grad_from_the_weight_grad_pass(oracle, shape, env, dtype):
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_bias_grad_tl
    M, K, N, H, BK, BN = shape
    _say("weight+bias grad", shape, env, dtype)
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=11)
    with _lib.tuning(**env):
        dhw, dbias = rz_linear_backward_weight_bias_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024),
                                                            BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert dhw.shape == (H,) and dhw.dtype == dtype
    assert dbias.shape == (N,) and dbias.dtype == dtype
    assert rel_err(dhw.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5)) <= TOL[dtype]
    # the bias gradient is not scaled by init_factor
    assert rel_err(dbias.float().cpu().numpy(), dy64.sum(axis=0)) <= TOL[dtype]


@pytest.mark.parametrize("out_dtype", ["same", "f32"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=_dt_id)
@pytest.mark.parametrize("env", [{}, {"lds_image": -1}, {"lds_image": -1, "fold": -1}], ids=_env_id)
@pytest.mark.parametrize("shape", CASES[:4], ids=_shape_id)
def test_accumulate_into_an_existing_gradient(oracle, tuned, shape, env, dtype, out_dtype):
    from rzlinear_amd.impl.RzLinearBackward import (rz_linear_backward_weight_bias_grad_tl,
                                                    rz_linear_backward_weight_grad_tl)
    tuned(**env)
    M, K, N, H, BK, BN = shape
    _say("accumulate", shape, env, dtype, out_dtype)
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=12)
    odt = torch.float32 if out_dtype == "f32" else dtype
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 1.0)
    g = torch.Generator().manual_seed(5)
    start = (torch.randn((H,), generator=g) * float(np.abs(ref).max())).to(odt)
    # overwrite into a caller-owned buffer
    buf = start.clone().cuda()
    out = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                            BLOCK_SIZE_N=BN, out=buf)
    torch.cuda.synchronize()
    assert out.data_ptr() == buf.data_ptr() and out.dtype == odt
    assert rel_err(buf.float().cpu().numpy(), ref) <= TOL[dtype]
    # add to what the buffer holds; twice, with the bias gradient the second time
    buf = start.clone().cuda()
    rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                      BLOCK_SIZE_N=BN, out=buf, accumulate=True)
    torch.cuda.synchronize()
    want = start.double().numpy() + ref
    assert rel_err(buf.float().cpu().numpy(), want) <= TOL[odt if odt != torch.float32 else dtype]
    _, dbias = rz_linear_backward_weight_bias_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                                      BLOCK_SIZE_N=BN, out=buf, accumulate=True)
    torch.cuda.synchronize()
    want = start.double().numpy() + 2 * ref
    assert rel_err(buf.float().cpu().numpy(), want) <= 2 * TOL[odt if odt != torch.float32 else dtype]
    assert rel_err(dbias.float().cpu().numpy(), dy64.sum(axis=0)) <= TOL[dtype]


def test_ex_argument_checks():
    import ctypes
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    lib = _lib.load()
    M, K, N, H = 64, 64, 64, 5000
    x = torch.zeros((M, K), device="cuda")
    dy = torch.zeros((M, N), device="cuda")
    dhw = torch.zeros((H,), device="cuda")
    R = (ctypes.c_int32 * 8)(*R1024)
    s = torch.cuda.current_stream().cuda_stream
    need = lib.rz_weight_grad_ex_workspace_bytes(M, K, N, H, 64, 64, 0, 0, 1)
    assert need > lib.rz_weight_grad_ex_workspace_bytes(M, K, N, H, 64, 64, 0, 0, 0)
    assert lib.rz_weight_grad_ex_workspace_bytes(M, K, N, H, 64, 64, 0, 0, 0) == \
        lib.rz_weight_grad_workspace_bytes(M, K, N, H, 64, 64, 0)
    # unknown flag bit, workspace too small for the column sums
    assert lib.rz_weight_grad_ex(x.data_ptr(), dy.data_ptr(), dhw.data_ptr(), None, None, 0, M, K, N, H, 64, 64,
                                 R, 1.0, K, N, 0, 8, s) == -9
    ws = torch.empty((need,), dtype=torch.uint8, device="cuda")
    dbias = torch.zeros((N,), device="cuda")
    assert lib.rz_weight_grad_ex(x.data_ptr(), dy.data_ptr(), dhw.data_ptr(), dbias.data_ptr(), ws.data_ptr(),
                                 need - 1, M, K, N, H, 64, 64, R, 1.0, K, N, 0, 0, s) == -7
    with pytest.raises(ValueError):
        rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=64,
                                          BLOCK_SIZE_N=64, accumulate=True)
    with pytest.raises(TypeError):
        rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=64,
                                          BLOCK_SIZE_N=64, out=torch.zeros((H,), device="cuda", dtype=torch.float16))


FOLD_CASES = [
    # (M, K, N, H, BK, BN, forced C tile)
    (40, 4096, 8192, 200000, 64, 64, 256),     # seven windows of hashed_weight, 36 shares of the 8192 tiles
    (48, 4096, 4096, 70000, 64, 64, 128),
    (64, 2048, 4096, 70000, 32, 64, 0),        # the reference's default hashed tile: two loads per tile and thread
    (300, 200, 330, 90000, 32, 64, 128),       # ragged in M, K and N: whole tiles are stored, zeros beyond K x N
    (520, 264, 328, 90000, 64, 32, 256),       # the C tile reaches beyond the grid of hashed tiles
    (2100, 512, 384, 50000, 128, 64, 128),     # M cut into slices: a list entry per (tile, slice); eight loads
    (200, 256, 512, 40000, 16, 64, 64),        # 16-row hashed tiles, 64 C tile
    (130, 300, 200, 37000, 16, 16, 0),         # tiles smaller than the workgroup: 256 of 1024 threads have an element
    (96, 512, 768, 60000, 128, 128, 256),      # sixteen loads per tile and thread
    (70, 1024, 1024, 1 << 20, 32, 32, 0),      # 32 windows; one load per tile and thread
    # hashed tiles that reach beyond K x N, and beyond the C tiles that were computed (what they
    # hold there was never written and must not be read); offsets confined to a few values
    (32, 64, 776, 20000, 128, 128, 0),
    (100, 16, 264, 2065, 128, 16, 0),
    (512, 1024, 264, 16385, 128, 128, 0),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=_dt_id)
@pytest.mark.parametrize("kernel", [1, 2], ids=["auto", "windowed"])
@pytest.mark.parametrize("shape", FOLD_CASES, ids=_shape_id)
def test_tiles_stored_plainly_and_folded_into_the_gradient(oracle, tuned, shape, kernel, dtype):
    """hashed_weight too large for an LDS image: the contraction kernel stores X^T.dY tile by tile
    and scatters nothing; the fold kernel's workgroups own windows of hashed_weight and add up the
    tiles that land there.  No atomics, a fixed order of additions: the same bits on every call.
    With the bias gradient, and accumulating into an existing buffer."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import (rz_linear_backward_weight_bias_grad_tl,
                                                    rz_linear_backward_weight_grad_tl)
    M, K, N, H, BK, BN, tile = shape
    # (fold = 1 leaves layers of at most 4096 tiles to the kernel for few tiles, fold = 2 sends them through
    #  the windowed kernel as well)
    tuned(fold=kernel, window=-1, lds_image=-1, tile=tile)
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    plan = _lib.plan_query(2, M, K, N, H, BK, BN, code)
    _say("fold", shape, dtype, plan)
    assert plan["mode"] == "fold", plan
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=67)
    kw = dict(BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5)
    a = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw)
    b, dbias = rz_linear_backward_weight_bias_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw)
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy()
    assert rel_err(f(a), ref) <= TOL[dtype]
    assert (f(a)[ref == 0] == 0).all()                 # slots that no tile covers are exactly zero
    assert rel_err(f(dbias), dy64.sum(axis=0)) <= TOL[dtype]
    assert torch.equal(a, b)
    assert torch.equal(a, rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw))
    start = torch.linspace(-1, 1, H).cuda()
    buf = start.clone()
    rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), out=buf, accumulate=True, **kw)
    torch.cuda.synchronize()
    assert rel_err(buf.cpu().numpy(), start.double().cpu().numpy() + ref) <= TOL[dtype]
    # and the atomic scatter agrees
    tuned(fold=-1, window=-1, lds_image=-1, tile=tile)
    assert _lib.plan_query(2, M, K, N, H, BK, BN, code)["mode"] == "atomics"
    c = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw)
    torch.cuda.synchronize()
    assert rel_err(f(c), ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=_dt_id)
@pytest.mark.parametrize("shape", [(1024, 512, 768, 70000, 64, 64), (4100, 320, 200, 300000, 32, 64),
                                   (300, 1000, 1100, 1 << 20, 16, 16)], ids=_shape_id)
def test_tiles_stored_in_the_layers_dtype_cost_one_rounding_each(oracle, tuned, shape, dtype):
    """A 16-bit layer with a 16-bit dHW keeps the tiles of X^T.dY for the fold in its own dtype (half the
    bytes).  Every stored value is a complete fp32 sum over M (or a slice of it), rounded once; the fold adds
    the values of a slot up in fp32: so the error of an element is bounded by one rounding of each of its
    addends plus the output's own — checked element by element against the oracle with exactly that
    allowance.  rz_tuning.fold_tiles = -1, and an fp32 dHW (RZ_WG_DHW_F32), keep fp32 tiles: one rounding
    in all, the element-wise bound without any allowance.  Same bits on every call either way."""
    from helpers import assert_close, stored_tiles_slack
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    M, K, N, H, BK, BN = shape
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=83)
    kw = dict(BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5)
    f = lambda t: t.float().cpu().numpy()
    lib = _lib.load()
    for kernel in (1, 2):   # the kernel for few tiles where it applies, and the windowed one
        tuned(fold=kernel, window=-1, lds_image=-1)
        plan = _lib.plan_query(2, M, K, N, H, BK, BN, code)
        _say("tiles in the layer's dtype", shape, dtype, plan)
        assert plan["mode"] == "fold", plan
        narrow_ws = lib.rz_weight_grad_hashed_workspace_bytes(M, K, N, H, BK, BN, code, 0, 0, ctypes.byref(_lib.Tuning(fold=kernel, window=-1, lds_image=-1)))
        a = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw)
        a2 = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw)
        slack = stored_tiles_slack(oracle, x64, dy64, shape, R1024, 0.5, dtype)
        assert slack is not None
        assert_close(f(a), ref, dtype, "dHW (tiles in the layer's dtype)", slack=slack)
        assert torch.equal(a, a2)
        tuned(fold=kernel, window=-1, lds_image=-1, fold_tiles=-1)
        wide_ws = lib.rz_weight_grad_hashed_workspace_bytes(M, K, N, H, BK, BN, code, 0, 0, ctypes.byref(_lib.Tuning(fold=kernel, window=-1, lds_image=-1, fold_tiles=-1)))
        assert wide_ws > narrow_ws
        b = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw)
        assert_close(f(b), ref, dtype, "dHW (fp32 tiles)")
        # an fp32 gradient buffer never goes through 16-bit tiles
        tuned(fold=kernel, window=-1, lds_image=-1)
        c = torch.zeros((H,), dtype=torch.float32, device="cuda")
        rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), out=c, **kw)
        torch.cuda.synchronize()
        assert_close(f(c), ref, torch.float32, "dHW (fp32 buffer)")


def test_fold_shares_take_a_partition_of_a_window_even_when_their_lists_overflow(oracle):
    """768 x 768 hashed tiles of 16 x 16 over a hashed_weight of 500 000: sixteen windows, sixteen
    workgroups to a window, and every one of them has more tiles (about 2 400) than its list holds
    (2 048 runs), so each works through its part in several chunks.  The parts must still be a
    partition of the window's tiles: a tile taken twice or dropped shows as an error of the size of
    the gradient itself.  Reference as in test_gpu_full_size.py (index map checked against the
    oracle, float64 product and index_add_ on the GPU)."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    from rzlinear_amd.impl.RzLinearIdx import rz_linear_weight_tl
    M, K, N, H, BK, BN = 32, 12288, 12288, 500000, 16, 16
    dtype = torch.bfloat16
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    plan = _lib.plan_query(2, M, K, N, H, BK, BN, code, planned=True)
    _say("fold, lists that overflow", plan)
    assert plan["mode"] == "fold" and plan["shares"] > 1
    tiles_per_share = (K // BK) * (N // BN) * (H / plan["windows"] + BK * BN) / H / plan["shares"]
    assert tiles_per_share * plan["slices"] > 2048          # more than a list holds
    g = torch.Generator().manual_seed(91)
    x = torch.randn((M, K), generator=g).to(dtype).cuda()
    dy = torch.randn((M, N), generator=g).to(dtype).cuda()
    kw = dict(BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    idx = rz_linear_weight_tl(torch.arange(H, dtype=torch.float32, device="cuda"), K, N, H, *rargs(R1024), **kw).long()
    assert np.array_equal(idx.cpu().numpy(), oracle.index_map(K, N, H, BK, BN, R1024))
    a = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), **kw)
    b = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), **kw)
    torch.cuda.synchronize()
    dW = x.double().t() @ dy.double()
    ref = torch.zeros((H,), dtype=torch.float64, device="cuda").index_add_(0, idx.reshape(-1), dW.reshape(-1))
    err = float((a.double() - ref).abs().max() / ref.abs().max())
    assert err <= TOL[dtype], err
    assert abs(float(a.double().sum() - dW.sum())) <= TOL[dtype] * float(dW.abs().sum()) / 10   # every tile exactly once
    assert torch.equal(a, b)


PLANNED_FOLDS = [
    # (M, K, N, H, BK, BN, dtype)
    (64, 4096, 4096, 300000, 16, 16, torch.bfloat16),      # 65536 tiles; ten windows, 25 workgroups to a window
    (48, 4800, 4800, 500000, 16, 16, torch.float32),       # 90000 tiles: more than one listing pass of the search
    (1000, 700, 1100, 2000000, 128, 128, torch.float32),   # runs of a tile in several list entries; tiles beyond K x N
    (2100, 1000, 900, 600000, 64, 64, torch.bfloat16),     # M in slices: several list entries per tile; 16-bit tiles
    (128, 2048, 2048, 9000000, 32, 64, torch.float16),     # whole rounds of 256 windows, no shares
]


@pytest.mark.parametrize("shape", PLANNED_FOLDS, ids=lambda s: "x".join(str(v) for v in s[:6]))
def test_fold_lists_of_a_layer_plan_give_the_bits_of_the_search(oracle, tuned, shape):
    """With a layer plan the fold kernel's workgroups read their windows' tiles from the plan's lists; without
    one they look for them among all tile offsets.  The lists hold the tiles in the order in which the search
    numbers them, so the additions happen in the same order: the same bits, also where a window is shared by
    several workgroups, where a workgroup's part overflows its list, and where a tile has several entries."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import weight_grad_hashed
    M, K, N, H, BK, BN, dtype = shape
    tuned(fold=1, window=-1)
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    plan = _lib.plan_query(2, M, K, N, H, BK, BN, code, planned=True)
    _say("fold lists", shape, plan)
    assert plan["mode"] == "fold"
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=72)
    R = _lib.hash_constants(*rargs(R1024))
    outs = []
    for planned in (False, True, True):
        outs.append(weight_grad_hashed(x, dy, 0.5, M, K, N, H, R, BK, BN, use_layer_plan=planned)[0])
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5)
    assert rel_err(outs[1].float().cpu().numpy(), ref) <= TOL[dtype]


SMALL_LAYERS = [
    # (M, K, N, H, BK, BN): a hashed_weight beyond an LDS image, at most 4096 tiles
    (1024, 1024, 1024, 65536, 64, 64),     # the reference's CPU-runnable configuration
    (128, 1024, 1024, 65536, 32, 64),      # its benchmark grid at K = N = 1024, the launchers' default tile
    (300, 200, 330, 250000, 32, 64),       # ragged; a thousand workgroups, most of them with no tile at all
    (4100, 192, 160, 50000, 64, 64),       # M in slices
    (77, 520, 264, 40000, 128, 128),       # tiles that reach beyond K x N
    (64, 4096, 4096, 1 << 18, 64, 64),     # 4096 tiles over 2^18 elements: the most this kernel takes
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=_dt_id)
@pytest.mark.parametrize("shape", SMALL_LAYERS, ids=_shape_id)
def test_small_layers_with_a_large_hashed_weight_are_folded_without_atomics(oracle, shape, dtype):
    """No tuning: a layer of few tiles whose hashed_weight does not fit an LDS image stores X^T.dY tile
    by tile and a second, small kernel adds the tiles up in a fixed order — the same bits on every call,
    where the atomic scatter it replaces left the order of the additions open.  With a layer plan's
    offsets and with the kernel's own hashing; accumulating; against the oracle."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl, weight_grad_hashed
    M, K, N, H, BK, BN = shape
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    plan = _lib.plan_query(2, M, K, N, H, BK, BN, code)
    _say("small fold", shape, dtype, plan)
    assert plan["mode"] == "fold" and plan["shares"] == 1
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=68)
    kw = dict(BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5)
    a = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw)
    b = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), **kw)
    R = _lib.hash_constants(*rargs(R1024))
    c, _ = weight_grad_hashed(x, dy, 0.5, M, K, N, H, R, BK, BN, use_layer_plan=False)
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy()
    assert rel_err(f(a), ref) <= TOL[dtype]
    assert (f(a)[ref == 0] == 0).all()
    assert torch.equal(a, b) and torch.equal(a, c)
    start = torch.linspace(-1, 1, H).cuda()
    buf = start.clone()
    rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), out=buf, accumulate=True, **kw)
    torch.cuda.synchronize()
    assert rel_err(buf.cpu().numpy(), start.double().cpu().numpy() + ref) <= TOL[dtype]
