"""GPU parity: the HIP kernels, called through the launchers (ctypes -> C ABI), against the
CPU oracle on the same seeded inputs."""
import sys

import numpy as np
import pytest
import torch

from helpers import SEED_CONSTANTS, TOL, assert_close, make_inputs, rargs, rel_err, stored_tiles_slack

pytestmark = pytest.mark.gpu

R1024 = SEED_CONSTANTS[1024]

# (M, K, N, H, BK, BN)
SHAPES = [
    (128, 128, 128, 65536, 64, 64),       # one workgroup tile, no edges
    (256, 512, 384, 20000, 32, 64),       # reference default tile
    (50, 100, 150, 5000, 32, 64),         # ragged everywhere, not multiples of the vector width
    (1, 16, 16, 300, 16, 16),             # smallest tile, single row
    (333, 257, 129, 40000, 64, 32),       # odd sizes, tile of the reference's weight-grad test
    (200, 1024, 256, 70000, 32, 128),     # tile of the reference's idx test
    (192, 300, 520, 70000, 128, 128),
    (64, 600, 200, 9000, 256, 16),
    (96, 96, 700, 9000, 16, 256),
    (1024, 1024, 1024, 65536, 64, 64),    # the reference's CPU-path configuration
]
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_forward(oracle, shape, dtype):
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
    M, K, N, H, BK, BN = shape
    _say("forward", shape, dtype)
    (x, hw, _), (x64, hw64, _) = make_inputs(M, K, N, H, dtype, seed=1)
    y = rz_linear_forward_tl(x, hw, 0.75, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert y.shape == (M, N) and y.dtype == dtype
    ref = oracle.forward(x64, hw64, N, BK, BN, R1024, 0.75)
    assert rel_err(y.float().cpu().numpy(), ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_input_grad(oracle, shape, dtype):
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_input_grad_tl
    M, K, N, H, BK, BN = shape
    _say("input_grad", shape, dtype)
    (_, hw, dy), (_, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=2)
    dx = rz_linear_backward_input_grad_tl(dy, hw, 1.25, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                          BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert dx.shape == (M, K) and dx.dtype == dtype
    ref = oracle.input_grad(dy64, hw64, K, BK, BN, R1024, 1.25)
    assert rel_err(dx.float().cpu().numpy(), ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_weight_grad(oracle, shape, dtype):
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_weight_grad_tl
    M, K, N, H, BK, BN = shape
    _say("weight_grad", shape, dtype)
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=3)
    dhw = rz_linear_backward_weight_grad_tl(x, dy, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK,
                                            BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert dhw.shape == (H,) and dhw.dtype == dtype
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5)
    assert rel_err(dhw.float().cpu().numpy(), ref) <= TOL[dtype]
    # slots that no tile covers stay exactly zero
    untouched = np.ones(H, dtype=bool)
    untouched[np.unique(oracle.index_map(K, N, H, BK, BN, R1024))] = False
    assert (dhw.float().cpu().numpy()[untouched] == 0).all()


@pytest.mark.parametrize("cfg", [
    (1024, 1024, 65536, 64, 64), (4096, 4096, 16778, 64, 64), (512, 1024, 5243, 64, 64),
    (4096, 16384, 67109, 64, 64), (2048, 2048, 32768, 64, 64), (1000, 77, 20000, 32, 64),
    (99999, 16, 300, 16, 16)], ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("levels", [1, 2])
def test_device_tile_offsets_bit_exact(oracle, cfg, levels):
    import ctypes
    from rzlinear_amd import _lib
    K, N, H, BK, BN = cfg
    _say("tile_offsets", cfg, levels)
    lib = _lib.load()
    TK, TN = -(-K // BK), -(-N // BN)
    for seed, R in SEED_CONSTANTS.items():
        out = torch.empty((TK, TN), dtype=torch.int32, device="cuda")
        _lib.check(lib.rz_tile_offsets_device(out.data_ptr(), K, N, H, BK, BN, (ctypes.c_int32 * 8)(*R),
                                              levels, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        ref = oracle.c_tile_offsets(K, N, H, BK, BN, R, levels)
        assert np.array_equal(out.cpu().numpy().astype(np.int64), ref)
        host = _lib.tile_offsets(K, N, H, BK, BN, R, levels).numpy().astype(np.int64)
        assert np.array_equal(host, ref)


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
def test_materialize_both_hashes(oracle, dtype):
    from rzlinear_amd.impl.RzLinearIdx import rz_linear_idx_tl, rz_linear_weight_tl
    K, N, H, BK, BN = 1024, 1024, 65536, 32, 128
    _say("materialize", dtype)
    hw = torch.arange(H).to(dtype).cuda() if dtype == torch.float32 else torch.randn(H).to(dtype).cuda()
    hw64 = hw.double().cpu().numpy()
    R = R1024
    w1 = rz_linear_idx_tl(hw, K, N, H, R[3], R[2], R[1], R[0], BK, BN)
    assert np.array_equal(w1.double().cpu().numpy(), oracle.materialize(hw64, K, N, BK, BN, R, 1))
    w2 = rz_linear_weight_tl(hw, 1000, 900, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    assert np.array_equal(w2.double().cpu().numpy(), oracle.materialize(hw64, 1000, 900, BK, BN, R, 2))


TILE_CASES = [
    # (M, K, N, H, BK, BN): complete tiles for every C-tile size, ragged, and both scatter paths
    (512, 512, 512, 9000, 64, 64),
    (300, 200, 330, 9000, 32, 64),
    (256, 256, 512, 70000, 64, 64),      # H too large for the LDS image: tiles stored and folded (fold = -1: global atomics)
    (130, 70, 90, 2000, 16, 16),         # 16-wide tiles: LDS atomics inside the image
    (2688, 192, 2432, 30000, 64, 64),    # > 384 tiles of 128: the four-wavefront 128 form
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("env", [{"tile": 32}, {"tile": 64}, {"tile": 128}, {"tile": 256}, {"tile": 128, "stages": 1},
                                 {"tile": 256, "lds_image": -1}, {"lds_image": -1, "fold": -1, "window": -1}],
                         ids=lambda e: "-".join("%s=%s" % (k, v) for k, v in e.items()))
@pytest.mark.parametrize("shape", TILE_CASES, ids=lambda s: "x".join(map(str, s)))
def test_every_tile_shape_and_scatter_mode(oracle, shape, env, dtype):
    """The library picks its C tile and scatter path from the problem size; force each one
    (rz_tuning overrides)."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_tl
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
    M, K, N, H, BK, BN = shape
    _say("tiles", shape, env, dtype)
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=4)
    with _lib.tuning(**env):
        y = rz_linear_forward_tl(x, hw, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        dx, dhw = rz_linear_backward_tl(x, hw, dy, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert rel_err(y.float().cpu().numpy(), oracle.forward(x64, hw64, N, BK, BN, R1024)) <= TOL[dtype]
    assert rel_err(dx.float().cpu().numpy(), oracle.input_grad(dy64, hw64, K, BK, BN, R1024)) <= TOL[dtype]
    assert rel_err(dhw.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R1024)) <= TOL[dtype]


@pytest.mark.parametrize("split", [0, -1], ids=["cut", "whole"])
@pytest.mark.parametrize("shape", [(32, 1536, 2048, 200000, 64, 64), (17, 100, 150, 5000, 32, 64),
                                   (8, 4096, 320, 70000, 64, 64), (32, 10240, 1024, 1 << 20, 64, 64),
                                   (1, 64, 64, 8192, 64, 64), (96, 2048, 4096, 300000, 32, 64),
                                   (150, 1000, 2100, 70000, 64, 64)], ids=lambda s: "x".join(map(str, s)))
def test_fp32_batches_of_at_most_32_rows_take_the_32_row_tile(oracle, shape, split):
    """The 32 x 64 tile of fp32 forward / input-grad (where a 64-row tile would be half padding:
    M <= 32, 65..96, 129..160, ...; large problems choose it by themselves), with and without a
    cut contraction, with a bias; also several tile rows, the last one ragged."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_input_grad_tl
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_bias_tl
    M, K, N, H, BK, BN = shape
    _say("32-row tile", shape, split)
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, torch.float32, seed=12)
    bias = torch.randn((N,), generator=torch.Generator().manual_seed(3))
    tn = dict(split=split) if split else {}
    with _lib.tuning(tile=32, **tn):
        assert _lib.plan_query(1, M, K, N, H, BK, BN, _lib.RZ_F32)["tile"] == 32
        y = rz_linear_forward_bias_tl(x, hw, bias.cuda(), 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        dx = rz_linear_backward_input_grad_tl(dy, hw, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    ref = oracle.forward(x64, hw64, N, BK, BN, R1024, 0.5) + bias.double().numpy()[None, :]
    assert rel_err(y.cpu().numpy(), ref) <= TOL[torch.float32]
    assert rel_err(dx.cpu().numpy(), oracle.input_grad(dy64, hw64, K, BK, BN, R1024, 0.5)) <= TOL[torch.float32]


FINISH_CASES = [
    # (M, K, N, H, BK, BN, tile override or 0)
    (32, 10240, 1024, 1 << 20, 64, 64, 0),      # skinny forward: many slices of few tiles
    (128, 2048, 8192, 16384, 64, 64, 0),        # input-grad contracts 8192
    (1024, 10240, 10240, 6553600, 32, 64, 256), # the reference's large grid shape: 160 tiles of 256 in three slices
    (100, 3000, 500, 9000, 32, 64, 0),          # ragged tiles and a ragged last slice
    (300, 4100, 260, 70000, 64, 64, 128),
    (17, 5000, 150, 5000, 16, 16, 64),
]


def test_cut_contractions_on_many_streams_at_once(oracle):
    """The counters of the slices that finish their own tiles live in the library, divided among streams:
    launches on different streams may run at the same time and must not share a counter.  Twenty streams
    (more than the library keeps parts for: the rest take the second kernel) each run cut forward
    contractions of two shapes, again and again, with nothing between them; every output must have the bits
    of the two-kernel form computed alone on the default stream."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_bias_tl
    dtype = torch.bfloat16
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    cases = [(128, 10240, 10240, 6553600, 32, 64), (64, 4096, 4096, 50000, 64, 64)]   # three and four slices
    _say("cut contractions on many streams")
    work = []
    for c, (M, K, N, H, BK, BN) in enumerate(cases):
        q = _lib.plan_query(0, M, K, N, H, BK, BN, code)
        assert q["mode"] == "split" and q["shares"] == 1, q     # cut, and finished by the kernel itself
        (x, hw, _), _ = make_inputs(M, K, N, H, dtype, seed=50 + c)
        bias = torch.randn((N,), generator=torch.Generator().manual_seed(c)).to(dtype).cuda()
        kw = dict(BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        with _lib.tuning(finish=-1):
            want = rz_linear_forward_bias_tl(x, hw, bias, 0.5, M, K, N, H, *rargs(R1024), **kw)
        work.append((x, hw, bias, (M, K, N, H), kw, want))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(20)]
    outs = []
    for rep in range(6):
        for i, st in enumerate(streams):
            x, hw, bias, dims, kw, want = work[(i + rep) % 2]
            with torch.cuda.stream(st):
                outs.append((rz_linear_forward_bias_tl(x, hw, bias, 0.5, *dims, *rargs(R1024), **kw), want, i, rep))
    torch.cuda.synchronize()
    for y, want, i, rep in outs:
        assert torch.equal(y, want), (i, rep)


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("case", FINISH_CASES, ids=lambda s: "x".join(map(str, s)))
def test_the_last_slice_to_arrive_finishes_the_tile(oracle, case, dtype):
    """A cut contraction (forward / input-grad of skinny problems) leaves no second kernel behind: the
    slices store their fp32 partial results, count themselves in at their tile, and the one that comes
    last adds the slices up in slice order — its own from its registers — adds the bias and stores.
    The bits are those of the two-kernel form (rz_tuning.finish = -1) whoever comes last; checked over
    several calls (the counters return to zero), with a bias, against the oracle."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_input_grad_tl
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_bias_tl
    M, K, N, H, BK, BN, tile = case
    shape = (M, K, N, H, BK, BN)
    _say("last slice finishes", case, dtype)
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=14)
    bias = torch.randn((N,), generator=torch.Generator().manual_seed(4)).to(dtype).cuda()
    kw = dict(BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    tn = dict(tile=tile) if tile else {}
    with _lib.tuning(**tn):
        plans = [_lib.plan_query(op, M, K, N, H, BK, BN, code) for op in (0, 1)]
    assert any(q["slices"] > 1 for q in plans) or dtype == torch.float32, plans
    if M >= 1024:   # (this case is finished by the kernel itself; the plans of the others may go to the second kernel)
        assert any(q["mode"] == "split" and q["shares"] == 1 for q in plans), plans
    # both forms on the SAME cut (the plan prices the two forms differently and may cut them differently): the
    # plan's own tile and slices where it cuts, three slices where it does not
    ys, dxs = [], []
    for op, q in enumerate(plans):
        same = dict(tile=q["tile"], split=q["slices"] if q["slices"] > 1 else 3)
        with _lib.tuning(**same):
            assert _lib.plan_query(op, M, K, N, H, BK, BN, code)["slices"] == same["split"]
            for _ in range(3):
                if op == 0:
                    ys.append(rz_linear_forward_bias_tl(x, hw, bias, 0.5, M, K, N, H, *rargs(R1024), **kw))
                else:
                    dxs.append(rz_linear_backward_input_grad_tl(dy, hw, 0.5, M, K, N, H, *rargs(R1024), **kw))
        with _lib.tuning(finish=-1, **same):
            assert _lib.plan_query(op, M, K, N, H, BK, BN, code)["slices"] == same["split"]
            if op == 0:
                y2 = rz_linear_forward_bias_tl(x, hw, bias, 0.5, M, K, N, H, *rargs(R1024), **kw)
            else:
                dx2 = rz_linear_backward_input_grad_tl(dy, hw, 0.5, M, K, N, H, *rargs(R1024), **kw)
    torch.cuda.synchronize()
    for y in ys:
        assert torch.equal(y, y2)
    for dx in dxs:
        assert torch.equal(dx, dx2)
    f = lambda t: t.float().cpu().numpy()
    assert_close(f(ys[0]), oracle.forward(x64, hw64, N, BK, BN, R1024, 0.5) + bias.double().cpu().numpy()[None, :], dtype, "Y")
    assert_close(f(dxs[0]), oracle.input_grad(dy64, hw64, K, BK, BN, R1024, 0.5), dtype, "dX")


def test_finishing_slices_read_what_this_launch_wrote():
    """The slice that finishes a tile reads the other slices' planes out of a workspace that earlier calls
    have filled with other values: alternating between two inputs over the same workspace, every call must
    give its own input's result (the bits of the two-kernel form), never a mixture with the call before."""
    import ctypes
    from rzlinear_amd import _lib
    lib = _lib.load()
    M, K, N, H, BK, BN = 256, 4096, 2048, 70000, 64, 64
    R = (ctypes.c_int32 * 8)(*R1024)
    stream = torch.cuda.current_stream().cuda_stream
    for dtype, code in ((torch.bfloat16, _lib.RZ_BF16), (torch.float32, _lib.RZ_F32)):
        fin = _lib.Tuning(tile=128, split=4)
        two = _lib.Tuning(tile=128, split=4, finish=-1)
        out = (ctypes.c_int32 * 8)()
        assert lib.rz_plan_query(0, M, K, N, H, BK, BN, code, 0, 0, ctypes.byref(fin), out) == 0 and (out[1], out[6]) == (4, 1)
        need = lib.rz_forward_hashed_workspace_bytes(M, K, N, H, BK, BN, code, ctypes.byref(fin))
        ws = torch.empty((need,), dtype=torch.uint8, device="cuda")
        inputs = [make_inputs(M, K, N, H, dtype, seed=s)[0] for s in (21, 22)]
        _say("finishing slices, alternating inputs", dtype)

        def forward(x, hw, tuning):
            y = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
            _lib.check(lib.rz_forward_hashed(x.data_ptr(), hw.data_ptr(), None, y.data_ptr(), ws.data_ptr(), need, M, K, N, H,
                                             BK, BN, R, 2, 1.0, K, N, code, ctypes.byref(tuning), stream))
            return y
        want = [forward(x, hw, two) for (x, hw, _) in inputs]
        torch.cuda.synchronize()
        assert not torch.equal(want[0], want[1])
        for i in range(8):
            x, hw, _ = inputs[i % 2]
            assert torch.equal(forward(x, hw, fin), want[i % 2]), (dtype, i)


@pytest.mark.parametrize("M", [32, 96, 160, 288])
def test_the_32_row_tile_is_chosen_where_64_rows_would_be_half_padding(oracle, M):
    """K = N = 4096, fp32: the plan takes the 32 x 64 tile by itself for these batch sizes (and not for
    M = 128 or 192), and the result matches the oracle."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_input_grad_tl
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
    K = N = 4096
    H, BK, BN = 1 << 20, 32, 64
    _say("32-row tile by plan", M)
    for op in (0, 1):
        assert _lib.plan_query(op, M, K, N, H, BK, BN, _lib.RZ_F32)["tile"] == 32
        assert _lib.plan_query(op, 128, K, N, H, BK, BN, _lib.RZ_F32)["tile"] != 32
        assert _lib.plan_query(op, 192, K, N, H, BK, BN, _lib.RZ_F32)["tile"] != 32
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, torch.float32, seed=14)
    y = rz_linear_forward_tl(x, hw, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    dx = rz_linear_backward_input_grad_tl(dy, hw, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), oracle.forward(x64, hw64, N, BK, BN, R1024, 1.0), torch.float32, "Y")
    assert_close(dx.cpu().numpy(), oracle.input_grad(dy64, hw64, K, BK, BN, R1024, 1.0), torch.float32, "dX")


def test_kernels_match_vectors_produced_by_the_reference_kernels():
    """fp32 HIP kernels against outputs of the reference's own Triton kernels on the same inputs
    (tests/golden/reference_vectors.npz)."""
    import os
    from rzlinear_amd.impl.RzLinearBackward import (rz_linear_backward_input_grad_tl,
                                                    rz_linear_backward_weight_grad_tl)
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz"))
    R = d["R"].tolist()
    for name in "abc":
        M, K, N, H, BK, BN = [int(v) for v in d[name + "_shape"]]
        f = float(d[name + "_f"])
        _say("reference vectors", name, (M, K, N, H, BK, BN))
        x, hw, dy = (torch.from_numpy(d[name + s]).cuda() for s in ("_x", "_hw", "_dy"))
        y = rz_linear_forward_tl(x, hw, f, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        dx = rz_linear_backward_input_grad_tl(dy, hw, f, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        dhw = rz_linear_backward_weight_grad_tl(x, dy, f, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        torch.cuda.synchronize()
        assert rel_err(y.cpu().numpy(), d[name + "_y"]) <= 1e-4
        assert rel_err(dx.cpu().numpy(), d[name + "_dx"]) <= 1e-4
        assert rel_err(dhw.cpu().numpy(), d[name + "_dhw"]) <= 1e-4


def test_fp16_kernels_match_fp16_vectors_produced_by_the_reference_kernels():
    """fp16 HIP kernels against the reference's own kernels on fp16 tensors
    (tests/golden/reference_vectors_16bit.npz).  Both accumulate the products in fp32 and round
    the output once, so they may differ by an fp16 rounding; the reference adds the weight
    gradient atomically in fp16, this build in fp32."""
    import os
    from rzlinear_amd.impl.RzLinearBackward import (rz_linear_backward_input_grad_tl,
                                                    rz_linear_backward_weight_grad_tl)
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors_16bit.npz"))
    R = d["R"].tolist()
    for name in "hi":
        M, K, N, H, BK, BN = [int(v) for v in d[name + "_shape"]]
        f = float(d[name + "_f"])
        _say("reference fp16 vectors", name, (M, K, N, H, BK, BN))
        x, hw, dy = (torch.from_numpy(d[name + s]).half().cuda() for s in ("_x", "_hw", "_dy"))
        y = rz_linear_forward_tl(x, hw, f, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        dx = rz_linear_backward_input_grad_tl(dy, hw, f, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        dhw = rz_linear_backward_weight_grad_tl(x, dy, f, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        torch.cuda.synchronize()
        assert rel_err(y.float().cpu().numpy(), d[name + "_y"]) <= 1e-3
        assert rel_err(dx.float().cpu().numpy(), d[name + "_dx"]) <= 1e-3
        assert rel_err(dhw.float().cpu().numpy(), d[name + "_dhw"]) <= 2e-3


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
def test_module_forward_backward_with_fused_bias(oracle, dtype):
    """The nn.Module end to end: N-D input, bias fused into the forward kernel, all gradients."""
    from rzlinear_amd import RzLinear
    B, S, K, N, BK, BN = 3, 50, 192, 130, 32, 64
    _say("module", dtype)
    g = torch.Generator().manual_seed(9)
    layer = RzLinear(K, N, seed=0, dtype=dtype, compress_ratio=0.5, init_factor=0.25, block_size_k=BK,
                     block_size_n=BN)
    H = layer._hashed_weight.shape[0]
    with torch.no_grad():
        layer._hashed_weight.copy_(((torch.rand(H, generator=g) * 2 - 1) / K ** 0.5).to(dtype))
        layer._bias.copy_(torch.randn(N, generator=g).to(dtype))
    layer = layer.cuda()
    x = torch.randn((B, S, K), generator=g).to(dtype).cuda().requires_grad_(True)
    dy = torch.randn((B, S, N), generator=g).to(dtype).cuda()
    y = layer(x)
    assert y.shape == (B, S, N) and y.dtype == dtype
    y.backward(dy)
    torch.cuda.synchronize()
    R = layer._random_numbers.tolist()
    assert R == SEED_CONSTANTS[0]
    x64 = x.detach().double().cpu().numpy().reshape(-1, K)
    dy64 = dy.double().cpu().numpy().reshape(-1, N)
    hw64 = layer._hashed_weight.detach().double().cpu().numpy()
    b64 = layer._bias.detach().double().cpu().numpy()
    tol = TOL[dtype]
    assert rel_err(y.detach().float().cpu().numpy().reshape(-1, N), oracle.forward(x64, hw64, N, BK, BN, R, 0.25) + b64) <= tol
    assert rel_err(x.grad.float().cpu().numpy().reshape(-1, K), oracle.input_grad(dy64, hw64, K, BK, BN, R, 0.25)) <= tol
    assert rel_err(layer._hashed_weight.grad.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R, 0.25)) <= tol
    assert rel_err(layer._bias.grad.float().cpu().numpy(), dy64.sum(0)) <= tol


def test_function_apply_with_the_reference_six_arguments(oracle):
    """RzLinearFunction.apply(input, hashed_weight, random_numbers, output_dim, chunk_size, init_factor)
    as reference code calls it: default tile from `controls`, no bias, and a gradient that is not
    needed is not computed."""
    from rzlinear_amd import RzLinearFunction, controls
    M, K, N, H = 70, 96, 128, 9000
    BK, BN = controls["block_size_k"], controls["block_size_n"]
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, torch.float32, seed=6)
    rnd = torch.tensor(R1024, dtype=torch.int32)
    hw.requires_grad_(True)
    y = RzLinearFunction.apply(x, hw, rnd, N, 1, 2.0)
    y.backward(dy)
    torch.cuda.synchronize()
    assert x.grad is None
    assert rel_err(y.detach().cpu().numpy(), oracle.forward(x64, hw64, N, BK, BN, R1024, 2.0)) <= 1e-4
    assert rel_err(hw.grad.cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 2.0)) <= 1e-4
    # shared hashed_weight: two layers, autograd adds their weight gradients
    hw2 = hw.detach().clone().requires_grad_(True)
    x2 = x.detach().clone().requires_grad_(True)
    out = RzLinearFunction.apply(x2, hw2, rnd, N, 1, 1.0) + RzLinearFunction.apply(x2, hw2, rnd, N, 1, 1.0)
    out.backward(dy)
    torch.cuda.synchronize()
    assert rel_err(hw2.grad.cpu().numpy(), 2 * oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 1.0)) <= 1e-4
    assert rel_err(x2.grad.cpu().numpy(), 2 * oracle.input_grad(dy64, hw64, K, BK, BN, R1024, 1.0)) <= 1e-4


@pytest.mark.parametrize("master", [False, True], ids=["grad", "main_grad_fp32"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
def test_layers_sharing_a_parameter_accumulate_inside_the_kernels(oracle, dtype, master):
    """Three RzLinear layers over ONE hashed_weight (python/rz_linear/RzLinear.py:54-58) with
    fuse_grad_accumulation: backward adds every layer's weight gradient into the parameter's
    gradient buffer inside the weight-grad kernels (no tensor per layer, no add over H by
    autograd).  Against the sum of the oracle's three gradients, and against the same network
    without the option."""
    import torch.nn as nn
    from rzlinear_amd import RzLinear
    dims = [(96, 160, 64, 64), (160, 128, 32, 64), (128, 72, 64, 32)]      # (K, N, BK, BN) per layer
    H, M = 30000, 200
    seeds = [3, 4, 5]
    g = torch.Generator().manual_seed(99)
    hw0 = ((torch.rand(H, generator=g) * 2 - 1) / 10).to(dtype)
    x0 = torch.randn((M, dims[0][0]), generator=g).to(dtype)
    dy0 = torch.randn((M, dims[-1][1]), generator=g).to(dtype)
    _say("shared parameter", dtype, "main_grad" if master else "grad")

    def run(fuse):
        hw = nn.Parameter(hw0.clone().cuda())
        if fuse and master:
            hw.main_grad = torch.zeros(H, dtype=torch.float32, device="cuda")
        layers = [RzLinear(K, N, hashed_weight=hw, seed=sd, bias=False, dtype=dtype, init_factor=0.5,
                           block_size_k=BK, block_size_n=BN, fuse_grad_accumulation=fuse)
                  for (K, N, BK, BN), sd in zip(dims, seeds)]
        x = x0.clone().cuda().requires_grad_(True)
        acts, h = [x], x
        for layer in layers:
            h = layer(h)
            acts.append(h)
        h.backward(dy0.cuda())
        torch.cuda.synchronize()
        grad = hw.main_grad if (fuse and master) else hw.grad
        return layers, [a.detach() for a in acts], x.grad, grad

    layers, acts, dx_fused, grad_fused = run(True)
    _, _, dx_plain, grad_plain = run(False)
    # oracle: chain the per-layer gradients through the recorded activations
    hw64 = hw0.double().numpy()
    up = dy0.double().numpy()
    want = np.zeros(H)
    for layer, (K, N, BK, BN), a in reversed(list(zip(layers, dims, acts[:-1]))):
        R = layer._random_numbers.tolist()
        want += oracle.weight_grad(a.double().cpu().numpy(), up, H, BK, BN, R, 0.5)
        up = oracle.input_grad(up, hw64, K, BK, BN, R, 0.5)
        up = torch.from_numpy(up).to(dtype).double().numpy()      # the kernels round dX to the layer dtype
    tol = TOL[dtype] * 2                                          # three layers' rounding on the way down
    assert grad_fused.dtype == (torch.float32 if master else dtype)
    assert rel_err(grad_fused.float().cpu().numpy(), want) <= tol
    assert rel_err(grad_plain.float().cpu().numpy(), want) <= tol
    assert rel_err(grad_fused.float().cpu().numpy(), grad_plain.float().cpu().numpy().astype(np.float64)) <= tol
    assert torch.equal(dx_fused, dx_plain)                        # the input gradient does not depend on the option
    # a second backward keeps adding into the same buffer
    before = grad_fused.clone()
    h = acts[0].clone().requires_grad_(True)
    out = h
    for layer in layers:
        out = layer(out)
    out.backward(dy0.cuda())
    torch.cuda.synchronize()
    now = layers[0]._hashed_weight.main_grad if master else layers[0]._hashed_weight.grad
    assert rel_err(now.float().cpu().numpy(), 2 * before.float().cpu().numpy().astype(np.float64)) <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
def test_empty_batch(dtype):
    """M = 0: the reference's launchers return an empty output / input gradient and a zero
    weight gradient (torch.zeros((0, N)), torch.zeros(H)); so do these, without a launch."""
    from rzlinear_amd import RzLinear
    layer = RzLinear(64, 96, dtype=dtype, compress_ratio=0.5, block_size_k=32, block_size_n=32).cuda()
    x = torch.zeros((0, 64), dtype=dtype, device="cuda", requires_grad=True)
    y = layer(x)
    assert y.shape == (0, 96) and y.dtype == dtype
    y.sum().backward()
    torch.cuda.synchronize()
    assert x.grad.shape == (0, 64)
    assert layer._hashed_weight.grad.shape == layer._hashed_weight.shape
    assert float(layer._hashed_weight.grad.abs().max()) == 0.0 and float(layer._bias.grad.abs().max()) == 0.0
    y3 = layer(torch.zeros((2, 0, 64), dtype=dtype, device="cuda"))
    assert y3.shape == (2, 0, 96)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", [(32, 2048, 1024, 70000, 32, 64), (100, 4096, 300, 20000, 64, 64),
                                   (7, 2100, 520, 9000, 16, 32)], ids=lambda s: "x".join(map(str, s)))
def test_skinny_problems_split_the_contraction(oracle, shape, dtype):
    """Few output tiles and a long contraction: forward / input-grad cut it into slices with fp32
    partial results (workspace) that a second kernel adds up, bias included."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_input_grad_tl
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_bias_tl
    M, K, N, H, BK, BN = shape
    _say("split", shape, dtype)
    lib = _lib.load()
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    assert lib.rz_forward_workspace_bytes(M, K, N, H, BK, BN, code) > 0      # these shapes do split
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=8)
    bias = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(dtype).cuda()
    y = rz_linear_forward_bias_tl(x, hw, bias, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    dx = rz_linear_backward_input_grad_tl(dy, hw, 0.5, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    ref_y = oracle.forward(x64, hw64, N, BK, BN, R1024, 0.5) + bias.double().cpu().numpy()
    assert rel_err(y.float().cpu().numpy(), ref_y) <= TOL[dtype]
    assert rel_err(dx.float().cpu().numpy(), oracle.input_grad(dy64, hw64, K, BK, BN, R1024, 0.5)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", [(1024, 4352, 2048, 70000, 128, 128), (1024, 2048, 4352, 70000, 128, 128),
                                   (1024, 2176, 2048, 300000, 256, 128), (1000, 4360, 2040, 70000, 128, 256)],
                         ids=lambda s: "x".join(map(str, s)))
def test_cut_contraction_on_the_long_step_tile(oracle, shape, dtype):
    """The 16-bit 128 tile in its eight-wavefront form walks the contraction in 128-element
    steps; a contraction cut into slices must cut on those steps, or a slice would start
    between two hashed tiles of 128 (or 256) rows and read offsets that nobody hashed.
    4352 = 34 x 128 and 2176 = 17 x 128 do not divide evenly over the slices."""
    from rzlinear_amd import _lib
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_input_grad_tl
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
    M, K, N, H, BK, BN = shape
    _say("cut contraction, long step", shape, dtype)
    code = _lib.dtype_code(torch.empty(0, dtype=dtype))
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=21)
    with _lib.tuning(tile=128):   # (the tile in question, whatever the plan would pick by itself; the cut stays the plan's)
        plans = [_lib.plan_query(op, M, K, N, H, BK, BN, code) for op in (0, 1)]
        assert any(p["tile"] == 128 and p["slices"] > 1 for p in plans), plans
        for p in plans:
            assert p["slices"] == 1 or p["slice_len"] % p["step"] == 0, p
        y = rz_linear_forward_tl(x, hw, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
        dx = rz_linear_backward_input_grad_tl(dy, hw, 1.0, M, K, N, H, *rargs(R1024), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert_close(y.float().cpu().numpy(), oracle.forward(x64, hw64, N, BK, BN, R1024), dtype, "Y")
    assert_close(dx.float().cpu().numpy(), oracle.input_grad(dy64, hw64, K, BK, BN, R1024), dtype, "dX")


def _random_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        BK, BN = (int(2 ** rng.integers(4, 9)) for _ in range(2))
        M, K, N = (int(rng.integers(1, 700)) for _ in range(3))
        if rng.random() < 0.3:      # complete tiles now and then, so the unchecked kernels run too
            M, K, N = (int(rng.choice([64, 128, 256, 512])) for _ in range(3))
        H = BK * BN + int(rng.integers(1, 60000))
        cases.append((M, K, N, H, BK, BN))
    return cases


@pytest.mark.parametrize("shape", _random_cases(40, 2024), ids=lambda s: "x".join(map(str, s)))
def test_random_shapes_fp32(oracle, shape):
    """Seeded random shapes, tiles and hashed sizes: every tile family, checked and unchecked
    kernels, split and unsplit contractions, LDS-image and atomic scatters get hit."""
    from rzlinear_amd.impl.RzLinearBackward import rz_linear_backward_tl
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_tl
    M, K, N, H, BK, BN = shape
    _say("random", shape)
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, torch.float32, seed=M + K + N)
    R = SEED_CONSTANTS[0]
    y = rz_linear_forward_tl(x, hw, 1.5, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    dx, dhw = rz_linear_backward_tl(x, hw, dy, 1.5, M, K, N, H, *rargs(R), BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), oracle.forward(x64, hw64, N, BK, BN, R, 1.5)) <= 1e-4
    assert rel_err(dx.cpu().numpy(), oracle.input_grad(dy64, hw64, K, BK, BN, R, 1.5)) <= 1e-4
    assert rel_err(dhw.cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R, 1.5)) <= 1e-4


def _random_cases_16bit(n, seed):
    """Shapes for the 16-bit kernels: larger than the fp32 sweep (so that the 128 and 256 tiles
    with direct staging are picked), mostly multiples of 8 (edge-clamped staging), some
    multiples of 64 or 256 (no bounds checks), some odd (bounds-checked register staging)."""
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        BK, BN = (int(2 ** rng.integers(4, 8)) for _ in range(2))
        kind = rng.random()
        if kind < 0.5:
            M, K, N = (8 * int(rng.integers(1, 160)) for _ in range(3))
        elif kind < 0.7:
            M, K, N = (64 * int(rng.integers(1, 20)) for _ in range(3))
        elif kind < 0.8:
            M, K, N = (256 * int(rng.integers(1, 5)) for _ in range(3))
        else:
            M, K, N = (int(rng.integers(1, 1300)) for _ in range(3))
        H = BK * BN + int(rng.integers(1, 120000))
        cases.append((M, K, N, H, BK, BN))
    return cases


@pytest.mark.parametrize("shape", _random_cases_16bit(40, 4242), ids=lambda s: "x".join(map(str, s)))
def test_random_shapes_16bit(oracle, shape):
    """Seeded random shapes for bf16 (even cases) and fp16 (odd cases), with the bias and the
    bias gradient in the same calls."""
    from rzlinear_amd.impl.RzLinearBackward import (rz_linear_backward_input_grad_tl,
                                                    rz_linear_backward_weight_bias_grad_tl)
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_bias_tl
    M, K, N, H, BK, BN = shape
    dtype = torch.bfloat16 if (M + K + N) % 2 == 0 else torch.float16
    _say("random 16-bit", shape, dtype)
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=M + 3 * K + 5 * N)
    bias = torch.linspace(-2, 2, N).to(dtype).cuda()
    R = SEED_CONSTANTS[0]
    kw = dict(BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    y = rz_linear_forward_bias_tl(x, hw, bias, 0.75, M, K, N, H, *rargs(R), **kw)
    dx = rz_linear_backward_input_grad_tl(dy, hw, 0.75, M, K, N, H, *rargs(R), **kw)
    dhw, dbias = rz_linear_backward_weight_bias_grad_tl(x, dy, 0.75, M, K, N, H, *rargs(R), **kw)
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy()
    assert_close(f(y), oracle.forward(x64, hw64, N, BK, BN, R, 0.75) + bias.double().cpu().numpy(), dtype, "Y")
    assert_close(f(dx), oracle.input_grad(dy64, hw64, K, BK, BN, R, 0.75), dtype, "dX")
    assert_close(f(dhw), oracle.weight_grad(x64, dy64, H, BK, BN, R, 0.75), dtype, "dHW",
                 slack=stored_tiles_slack(oracle, x64, dy64, shape, R, 0.75, dtype))
    assert_close(f(dbias), dy64.sum(axis=0), dtype, "dbias")


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", [(1100, 1023, 1001, 40000, 32, 64), (1030, 1025, 2047, 300000, 64, 64),
                                   (512, 1031, 1017, 9000, 64, 64), (300, 9, 15, 3000, 16, 16), (257, 2049, 263, 9000, 64, 64),
                                   (200, 5, 6, 3000, 16, 16), (4200, 1022, 1026, 16384, 64, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rows_that_are_not_whole_16_byte_pieces(oracle, shape, dtype):
    """K and N that are not multiples of 8 (of 4 for fp32), the operands contiguous (so that every row starts at another
    alignment and the last row ends with the allocation's last element): the kernels keep their
    direct-to-LDS path, fetch the piece that straddles a row end as it lies, and put the last row's
    right in LDS; nothing is copied or padded on the way (the reference masks element by element,
    python/rz_linear/impl/RzLinearForward.py:338-341).  Straight through the C ABI, all three
    products and the bias gradient against the oracle, element by element; a hashed_weight with an
    inf in a slot that no tile of the layer touches must not show in any result."""
    import ctypes
    from rzlinear_amd import _lib
    lib = _lib.load()
    M, K, N, H, BK, BN = shape
    _say("odd rows, in the kernels", shape, dtype)
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=31)
    # exact-size allocations: the row ends are where the tensors end
    x, dy = x.clone(), dy.clone()
    code = _lib.dtype_code(x)
    R = (ctypes.c_int32 * 8)(*R1024)
    stream = torch.cuda.current_stream().cuda_stream
    bias = torch.randn((N,), generator=torch.Generator().manual_seed(5)).to(dtype).cuda()
    # an inf where no tile reaches (if there is such a slot): the padded-copy scheme this replaces turned it into NaN
    idx = oracle.index_map(K, N, H, BK, BN, R1024)
    free = np.setdiff1d(np.arange(H), idx.reshape(-1))
    if free.size:
        hw[int(free[0])] = float("inf")
    y = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    dx = torch.full((M, K), float("nan"), dtype=dtype, device="cuda")
    dhw = torch.full((H,), float("nan"), dtype=dtype, device="cuda")
    dbias = torch.full((N,), float("nan"), dtype=dtype, device="cuda")
    fq = _lib.plan_query(0, M, K, N, H, BK, BN, code)
    _lib.check(lib.rz_forward_bias(x.data_ptr(), hw.data_ptr(), bias.data_ptr(), y.data_ptr(), M, K, N, H, BK, BN, R, 1.0,
                                   K, N, code, stream))
    _lib.check(lib.rz_input_grad(dy.data_ptr(), hw.data_ptr(), dx.data_ptr(), M, K, N, H, BK, BN, R, 1.0, N, K, code, stream))
    need = lib.rz_weight_grad_ex_workspace_bytes(M, K, N, H, BK, BN, code, 0, 1)
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device="cuda")
    _lib.check(lib.rz_weight_grad_ex(x.data_ptr(), dy.data_ptr(), dhw.data_ptr(), dbias.data_ptr(), ws.data_ptr(), need,
                                     M, K, N, H, BK, BN, R, 1.0, K, N, code, 0, stream))
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy()
    assert_close(f(y), oracle.forward(x64, hw64, N, BK, BN, R1024) + bias.double().cpu().numpy()[None, :], dtype, "Y")
    assert_close(f(dx), oracle.input_grad(dy64, hw64, K, BK, BN, R1024), dtype, "dX")
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024)
    assert_close(f(dhw), ref, dtype, "dHW", slack=stored_tiles_slack(oracle, x64, dy64, shape, R1024, 1.0, dtype))
    assert (f(dhw)[ref == 0] == 0).all()
    assert rel_err(f(dbias), dy64.sum(axis=0)) <= TOL[dtype]
    # (where the plan takes a 128 or 256 tile these shapes run the direct-to-LDS kernels: say which)
    _say("   forward plan", fq, "weight-grad plan", _lib.plan_query(2, M, K, N, H, BK, BN, code))
