"""GPU parity of the windowed weight-grad (large hashed_weight, short contraction): every
workgroup owns a range of dHW and pulls in the tiles that touch it.  rz_tuning.window = 1 forces
that path wherever it is possible; the last test lets the library choose it by itself."""
import sys

import numpy as np
import pytest
import torch

from helpers import SEED_CONSTANTS, TOL, make_inputs, rargs, rel_err

pytestmark = pytest.mark.gpu

R1024 = SEED_CONSTANTS[1024]

# (M, K, N, H, BK, BN): H too large for one LDS image in every case
CASES = [
    (256, 256, 512, 70000, 64, 64),
    (32, 1024, 1024, 65536, 64, 64),
    (50, 300, 330, 70000, 32, 64),        # ragged in M, K and N; the reference's default tile
    (200, 512, 512, 300000, 64, 64),      # 256 windows of about 1.2 K elements
    (31, 640, 640, 2000001, 64, 64),      # most of dHW untouched, odd H
    (130, 192, 128, 7000000, 64, 64),     # two rounds of windows; M spans several chunks
    (40, 520, 264, 500000, 64, 64),       # 16-byte pieces whole, last tile row has one strip beyond K
    (17, 96, 72, 100000, 32, 64),         # one partial group of rows of M
    (8, 4096, 8192, 40000, 64, 64),       # more strips meet a window than its list holds (16-bit)
    # the other hashed tiles of the reference's own tests (python/tests/test_rz_linear.py:38-39, :95-96) and of
    # its autotuner: 128 columns are two 64-column units side by side, 32 columns a narrower unit, up to 256 rows
    (48, 512, 1024, 300000, 32, 128),
    (100, 520, 200, 90000, 64, 32),       # ragged: the last tiles reach beyond K and N
    (33, 640, 768, 500000, 128, 128),
    (70, 300, 330, 70000, 128, 64),
    (20, 1024, 264, 200000, 256, 32),
    (24, 200, 520, 150000, 32, 128),      # N ends inside the first unit of the last tile: its second lies beyond N
    (16, 2048, 4096, 40000, 64, 32),      # more units meet a window than its list holds
    (45, 257, 259, 80000, 64, 128),       # rows that are not whole 16-byte pieces: fragments element by element
]
_dt_id = lambda d: str(d).split(".")[-1]
_shape_id = lambda s: "x".join(map(str, s))


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=_dt_id)
@pytest.mark.parametrize("shape", CASES, ids=_shape_id)
def test_windowed_weight_grad(oracle, tuned, monkeypatch, shape, dtype):
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    tuned(window=1)
    M, K, N, H, BK, BN = shape
    _say("windowed weight grad", shape, dtype)
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=31)
    # without a layer plan (every workgroup searches the tile offsets for its strips) ...
    monkeypatch.setattr(_lib, "use_layer_plans", False)
    dhw = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                            BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5)
    got = dhw.float().cpu().numpy()
    assert rel_err(got, ref) <= TOL[dtype]
    # ... and with one (the lists come from the plan): the same strips in the same order, the same bits
    monkeypatch.setattr(_lib, "use_layer_plans", True)
    _say("  with a layer plan")
    planned = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                                BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert torch.equal(planned, dhw)
    assert (got[ref == 0] == 0).all()          # slots that no tile covers stay exactly zero
    # the summation order is fixed: a second call gives the same bits
    again = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                              BLOCK_SIZE_N=BN)
    assert torch.equal(dhw, again)
    # and the scatter kernel agrees
    tuned(window=-1)
    scatter = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                                BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert rel_err(scatter.float().cpu().numpy(), ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=_dt_id)
def test_windowed_accumulate_and_fp32_buffer(oracle, tuned, dtype):
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    tuned(window=1)
    M, K, N, H, BK, BN = 64, 512, 256, 90000, 64, 64
    _say("windowed accumulate", dtype)
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=32)
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 1.0)
    for odt in (dtype, torch.float32):
        start = (torch.randn((H,), generator=torch.Generator().manual_seed(6)) * float(np.abs(ref).max())).to(odt)
        buf = start.clone().cuda()
        rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN,
                                          out=buf, accumulate=True)
        torch.cuda.synchronize()
        tol = TOL[odt if odt != torch.float32 else dtype]
        assert rel_err(buf.float().cpu().numpy(), start.double().numpy() + ref) <= tol
        buf = start.clone().cuda()
        rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN,
                                          out=buf)
        torch.cuda.synchronize()
        assert rel_err(buf.float().cpu().numpy(), ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=_dt_id)
def test_bias_gradient_beside_the_window_kernel(oracle, tuned, dtype):
    """A layer with a bias asks for dbias in the same call; the window kernel does not stage dY by
    tile columns, so the column sums come from a pass of their own and the window path is kept."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_bias_grad_tl
    tuned(window=1)
    M, K, N, H, BK, BN = 45, 384, 520, 200000, 64, 64
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    assert _lib.plan_query(2, M, K, N, H, BK, BN, code, 0, True)["mode"] == "window"
    _say("window + dbias", dtype)
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=35)
    dhw, dbias = rz_linear_backward_weight_bias_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                                        BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert rel_err(dhw.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5)) <= TOL[dtype]
    assert rel_err(dbias.float().cpu().numpy(), dy64.sum(axis=0)) <= TOL[dtype]


def test_library_picks_the_window_path_for_skinny_batches(oracle):
    """M = 32 against K = N = 4096 with a 2^20-element hashed_weight: no tuning override."""
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    M, K, N, H, BK, BN = 32, 4096, 4096, 1 << 20, 64, 64
    _say("window path chosen by the plan")
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, torch.bfloat16, seed=33)
    a = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    b = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert rel_err(a.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 1.0)) <= TOL[torch.bfloat16]
    assert torch.equal(a, b)   # deterministic, unlike the atomic scatter


def _random_window_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        BK = int(rng.choice([32, 64]))
        M = int(rng.integers(1, 300))
        K, N = (int(rng.integers(8, 1500)) for _ in range(2))
        H = int(rng.integers(40000, 3000000))
        cases.append((M, K, N, H, BK, 64))
    return cases


@pytest.mark.parametrize("shape", _random_window_cases(24, 777), ids=_shape_id)
def test_windowed_weight_grad_random_shapes(oracle, tuned, shape):
    """Seeded random shapes through the window kernel: fp32 for even M, bf16 for odd M."""
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    tuned(window=1)
    M, K, N, H, BK, BN = shape
    dtype = torch.float32 if M % 2 == 0 else torch.bfloat16
    _say("windowed random", shape, dtype)
    R = SEED_CONSTANTS[0]
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=M + K + N)
    dhw = rz_linear_backward_weight_grad_tl(x, dy, 1.25, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert rel_err(dhw.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R, 1.25)) <= TOL[dtype]


def test_a_plan_of_another_layer_is_refused_on_the_device(tuned):
    """The host can check a plan's size only; the kernel checks its header against the call and
    turns dHW into NaN instead of following lists that belong to other shapes."""
    from rzlinear_amd import _lib
    tuned(window=1)
    M, K, N, H, BK, BN = 32, 512, 512, 300000, 64, 64
    _say("foreign layer plan")
    (x, _, dy), _ = make_inputs(M, K, N, H, torch.float32, seed=41)
    lib = _lib.load()
    R = _lib.hash_constants(*rargs(R1024))
    plan = _lib.layer_plan(K, N, H, BK, BN, R, 2, x.device).clone()
    plan[2] = K + 64                                   # the header now names another K
    out = torch.zeros((H,), device=x.device)
    _lib.check(lib.rz_weight_grad_planned(x.data_ptr(), dy.data_ptr(), out.data_ptr(), None, None, 0, plan.data_ptr(),
                                          plan.numel() * 4, M, K, N, H, BK, BN, R, 2, 1.0, K, N, _lib.RZ_F32, 0,
                                          _lib.current_tuning(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.isnan(out).all()


@pytest.mark.parametrize("mode", ["window", "fold"])
def test_a_plan_built_with_other_hash_constants_is_refused_on_the_device(tuned, mode):
    """Same K, N, H and tile, other constants: every offset of the plan is in range and wrong.  The
    header carries a checksum of the constants; the window kernel and the fold kernel compare it
    with their call's and store NaN instead of a wrong gradient."""
    from rzlinear_amd import _lib
    tuned(window=1) if mode == "window" else tuned(fold=1, window=-1)
    M, K, N, H, BK, BN = 32, 512, 512, 300000, 64, 64
    _say("layer plan of other constants", mode)
    (x, _, dy), _ = make_inputs(M, K, N, H, torch.float32, seed=42)
    lib = _lib.load()
    R = _lib.hash_constants(*rargs(R1024))
    other = _lib.hash_constants(*rargs(SEED_CONSTANTS[0]))
    assert _lib.plan_query(2, M, K, N, H, BK, BN, _lib.RZ_F32, planned=True)["mode"] == mode
    need = lib.rz_weight_grad_hashed_workspace_bytes(M, K, N, H, BK, BN, _lib.RZ_F32, 0, 0, _lib.current_tuning())
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device=x.device)
    out = {}
    for name, consts in (("own", R), ("other", other)):
        plan = _lib.layer_plan(K, N, H, BK, BN, consts, 2, x.device)
        out[name] = torch.zeros((H,), device=x.device)
        _lib.check(lib.rz_weight_grad_planned(x.data_ptr(), dy.data_ptr(), out[name].data_ptr(), None, ws.data_ptr(), need,
                                              plan.data_ptr(), plan.numel() * 4, M, K, N, H, BK, BN, R, 2, 1.0, K, N,
                                              _lib.RZ_F32, 0, _lib.current_tuning(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.isfinite(out["own"]).all() and float(out["own"].abs().max()) > 0
    assert torch.isnan(out["other"]).all()


def test_a_wavefront_that_gives_up_waiting_spoils_its_window_and_leaves(oracle, tuned):
    """The wait for earlier strips is bounded.  With the bound set to one look (from the host, through
    rz_tuning) wavefronts give up where they would have waited: the kernel still ends, and every
    window of dHW is either exactly what the unbounded run gives or NaN throughout."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    M, K, N, H, BK, BN = 64, 1024, 1024, 200000, 64, 64
    _say("bounded wait of the window kernel")
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, torch.bfloat16, seed=44)
    code = _lib.dtype_code(x)
    tuned(window=1)
    q = _lib.plan_query(2, M, K, N, H, BK, BN, code, planned=True)
    assert q["mode"] == "window"
    good = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    tuned(window=1, poll_limit=1)
    hasty = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert rel_err(good.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 1.0)) <= TOL[torch.bfloat16]
    window = -(-H // q["windows"])
    window = (window + 3) // 4 * 4
    spoilt = 0
    for w0 in range(0, H, window):
        a, b = hasty[w0:w0 + window], good[w0:w0 + window]
        if torch.isnan(a).any():
            assert torch.isnan(a).all()
            spoilt += 1
        else:
            assert torch.equal(a, b)
    _say("  windows stored as NaN: %d of %d" % (spoilt, q["windows"]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=_dt_id)
def test_fold_path_takes_its_tile_offsets_from_the_plan(oracle, tuned, monkeypatch, dtype):
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    tuned(fold=1, window=-1)
    M, K, N, H, BK, BN = 300, 512, 768, 90000, 64, 64
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    assert _lib.plan_query(2, M, K, N, H, BK, BN, code)["mode"] == "fold"
    _say("fold with a layer plan", dtype)
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=43)
    monkeypatch.setattr(_lib, "use_layer_plans", False)
    a = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    monkeypatch.setattr(_lib, "use_layer_plans", True)
    b = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    assert rel_err(b.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 1.0)) <= TOL[dtype]
