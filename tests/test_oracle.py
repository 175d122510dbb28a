"""Pins the CPU oracle (oracle/rz_oracle.py + oracle/rz_oracle.c) without running any reference
code: hand-evaluated known answers, degenerate hashes, structural invariants, the identity-input
trick of the reference's notebooks, torch.autograd through a gather, brute force on tiny shapes,
and the two restatements against each other."""
import itertools
import json
import os

import numpy as np
import pytest
import torch

R1024 = [45007, 20011, 38363, 15263, 24507, 36489, 12234, 43027]
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ------------------------------------------------------------------ hash constants
def test_hash_constants_fixture_matches_torch_rng(oracle):
    fx = json.load(open(os.path.join(GOLDEN, "hash_constants.json")))
    state = torch.get_rng_state()
    try:
        for seed, want in fx["seeds"].items():
            torch.manual_seed(int(seed))
            got = [fx["P"]] + torch.randint(0, fx["P"], (7,)).tolist()
            assert got == want
            assert oracle.HASH_CONSTANTS[int(seed)] == want
    finally:
        torch.set_rng_state(state)


# ------------------------------------------------------------------ tile hash
# Worked by hand from the formula in RzLinearForward.py:316 with R of seed 1024:
#   (0,1): a = R2+R1 = 58374, hi = 58374-45007 = 13367; b = R5+R4 = 60996, lo = 15989;
#          v = 13367*45007 + 15989 = 601624558; 601624558 mod 61440 = 4078
KAT_TWO_LEVEL = [
    # (tk, tn, H, BK, BN, expected offset)
    (0, 0, 65536, 64, 64, 10624),
    (0, 1, 65536, 64, 64, 4078),
    (1, 0, 65536, 64, 64, 51285),
    (1, 1, 65536, 64, 64, 44739),
    (63, 63, 65536, 64, 64, 16786),
    (5, 17, 65536, 64, 64, 6597),
    (0, 0, 16778, 64, 64, 9308),
    (63, 63, 16778, 64, 64, 9232),
    (31, 7, 16778, 64, 64, 11971),
    (127, 15, 16778, 32, 64, 2928),
]
# RzLinearIdx.py:70-71 / the formula inside the reference's test_get_idx (test_rz_linear.py:26-27)
KAT_ONE_LEVEL = [(0, 0, 65536, 32, 128, 20011), (3, 2, 65536, 32, 128, 7505), (31, 7, 65536, 32, 128, 41593)]


@pytest.mark.parametrize("tk,tn,H,BK,BN,want", KAT_TWO_LEVEL)
def test_two_level_offset_known_answers(oracle, tk, tn, H, BK, BN, want):
    assert oracle.tile_offset(tk, tn, H, BK, BN, R1024) == want
    K, N = (tk + 1) * BK, (tn + 1) * BN
    assert oracle.c_tile_offsets(K, N, H, BK, BN, R1024)[tk, tn] == want
    assert oracle.tile_offsets(K, N, H, BK, BN, R1024)[tk, tn] == want


@pytest.mark.parametrize("tk,tn,H,BK,BN,want", KAT_ONE_LEVEL)
def test_one_level_offset_known_answers(oracle, tk, tn, H, BK, BN, want):
    assert oracle.tile_offset(tk, tn, H, BK, BN, R1024, hash_levels=1) == want
    assert oracle.c_tile_offsets((tk + 1) * BK, (tn + 1) * BN, H, BK, BN, R1024, 1)[tk, tn] == want


def test_offset_degenerate_cases(oracle):
    # range 1 => every offset is 0
    assert not oracle.c_tile_offsets(512, 512, 64 * 64 + 1, 64, 64, R1024).any()
    # no dependence on the tile => one constant: ((R1 % R0) * R0 + R4 % R0) % range
    R = [45007, 20011, 0, 0, 24507, 0, 999, 0]
    offs = oracle.c_tile_offsets(512, 512, 65536, 64, 64, R)
    assert (offs == (20011 * 45007 + 24507) % (65536 - 4096)).all() and offs[0, 0] == 10624
    # only tk matters when R2 = R5 = 0, only tn when R3 = R7 = 0
    R = list(R1024); R[2] = R[5] = 0
    offs = oracle.c_tile_offsets(512, 512, 65536, 64, 64, R)
    assert (offs == offs[:, :1]).all() and len(set(offs[:, 0])) > 1
    R = list(R1024); R[3] = R[7] = 0
    offs = oracle.c_tile_offsets(512, 512, 65536, 64, 64, R)
    assert (offs == offs[:1, :]).all() and len(set(offs[0, :])) > 1


def test_offset_structure(oracle):
    H, BK, BN = 16778, 64, 64
    base = oracle.c_tile_offsets(4096, 4096, H, BK, BN, R1024)
    # R6 takes part in no formula
    R = list(R1024); R[6] = 7
    assert np.array_equal(base, oracle.c_tile_offsets(4096, 4096, H, BK, BN, R))
    # every other constant matters
    for i in (1, 2, 3, 4, 5, 7):
        R = list(R1024); R[i] = (R[i] + 1) % 45007
        assert not np.array_equal(base, oracle.c_tile_offsets(4096, 4096, H, BK, BN, R)), i
    # both linear terms are reduced mod R0: shifting a tile index by R0 changes nothing
    for tk, tn in [(0, 0), (3, 9), (40, 2)]:
        assert oracle.tile_offset(tk + 45007, tn, H, BK, BN, R1024) == base[tk, tn]
        assert oracle.tile_offset(tk, tn + 45007, H, BK, BN, R1024) == base[tk, tn]
    # tk multiplies R3/R7 and tn multiplies R2/R5 (not the other way round): compare with the
    # formula evaluated on swapped constants
    Rs = list(R1024); Rs[2], Rs[3] = Rs[3], Rs[2]; Rs[5], Rs[7] = Rs[7], Rs[5]
    swapped = oracle.c_tile_offsets(4096, 4096, H, BK, BN, Rs)
    assert np.array_equal(swapped, base.T) and not np.array_equal(swapped, base)
    # range
    assert base.min() >= 0 and base.max() < H - BK * BN


@pytest.mark.parametrize("cfg", [(1024, 1024, 65536, 64, 64), (1024, 1024, 16384, 64, 64),
                                 (2048, 2048, 16384, 64, 64), (4096, 4096, 16778, 64, 64),
                                 (512, 1024, 5243, 64, 64), (4096, 16384, 67109, 64, 64),
                                 (2048, 2048, 32768, 64, 64), (4096, 4096, 16778, 32, 64),
                                 (1000, 77, 20000, 32, 64)])
def test_offsets_numpy_equals_c_and_fits_int32(oracle, cfg):
    K, N, H, BK, BN = cfg
    a = oracle.tile_offsets(K, N, H, BK, BN, R1024)
    b = oracle.c_tile_offsets(K, N, H, BK, BN, R1024)
    assert np.array_equal(a, b)
    assert a.min() >= 0 and a.max() < H - BK * BN
    # the reference evaluates in int32: the largest intermediates must fit
    TK, TN = a.shape
    assert TK * R1024[3] + TN * R1024[2] + R1024[1] < 2**31
    assert 45006 * 45007 + 45006 < 2**31


def test_c_oracle_rejects_bad_hash_inputs(oracle):
    with pytest.raises(ValueError):
        oracle.c_tile_offsets(64, 64, 4096, 64, 64, R1024)          # H == BK*BN
    big = [2**31 - 1] + R1024[1:]
    with pytest.raises(ValueError):
        oracle.c_tile_offsets(64, 64, 65536, 64, 64, big)           # (R0-1)*R0 overflows int32


# ------------------------------------------------------------------ materialise / index map
def test_index_map_is_tilewise_contiguous(oracle):
    K, N, H, BK, BN = 96, 160, 9000, 32, 64
    idx = oracle.index_map(K, N, H, BK, BN, R1024)
    offs = oracle.tile_offsets(K, N, H, BK, BN, R1024)
    for tk, tn in itertools.product(range(K // BK), range(-(-N // BN))):
        blk = idx[tk * BK:(tk + 1) * BK, tn * BN:(tn + 1) * BN]
        full = offs[tk, tn] + np.arange(BK * BN).reshape(BK, BN)
        assert np.array_equal(blk, full[:, :blk.shape[1]])
    hw = np.arange(H, dtype=np.float64)
    assert np.array_equal(oracle.materialize(hw, K, N, BK, BN, R1024), idx)
    assert np.array_equal(oracle.c_materialize(hw, K, N, BK, BN, R1024), idx)
    # one-level variant as in the reference's test_get_idx oracle (test_rz_linear.py:21-33)
    want = np.empty((K, N))
    for k in range(K // BK):
        for n in range(N // 32):
            o = ((k * R1024[3] + n * R1024[2] + R1024[1]) % R1024[0]) % (H - BK * 32)
            want[k * BK:(k + 1) * BK, n * 32:(n + 1) * 32] = hw[o:o + BK * 32].reshape(BK, 32)
    assert np.array_equal(oracle.c_materialize(hw, K, N, BK, 32, R1024, 1), want)
    assert np.array_equal(oracle.materialize(hw, K, N, BK, 32, R1024, 1), want)


def test_identity_input_reads_back_the_index_map(oracle):
    # the reference's notebooks: hashed_weight = arange(H), input = eye(K) => output = index map
    K, N, H, BK, BN = 64, 96, 3000, 16, 32
    hw = np.arange(H, dtype=np.float64)
    idx = oracle.index_map(K, N, H, BK, BN, R1024)
    for fwd in (oracle.forward, oracle.c_forward):
        Y = fwd(np.eye(K), hw, N, BK, BN, R1024, 2.0)
        assert np.array_equal(Y, 2.0 * idx)
        # inside a tile: +1 along n, +BN along k
        assert np.array_equal(np.diff(Y[:, :BN], axis=1), 2.0 * np.ones((K, BN - 1)))
        assert np.array_equal(np.diff(Y[:BK, :], axis=0), 2.0 * BN * np.ones((BK - 1, N)))


# ------------------------------------------------------------------ the three contractions
def _brute(X, hw, dY, K, N, H, BK, BN, R, f, oracle):
    """Element by element from the definition W[k,n] = hw[off(k//BK, n//BN) + (k%BK)*BN + n%BN]."""
    M = X.shape[0]
    W = np.zeros((K, N))
    for k in range(K):
        for n in range(N):
            W[k, n] = hw[oracle.tile_offset(k // BK, n // BN, H, BK, BN, R) + (k % BK) * BN + n % BN]
    Y = np.zeros((M, N)); dX = np.zeros((M, K)); dHW = np.zeros(H)
    for m in range(M):
        for k in range(K):
            for n in range(N):
                Y[m, n] += X[m, k] * W[k, n] * f
                dX[m, k] += dY[m, n] * W[k, n] * f
                dHW[oracle.tile_offset(k // BK, n // BN, H, BK, BN, R) + (k % BK) * BN + n % BN] += \
                    X[m, k] * dY[m, n] * f
    return Y, dX, dHW


@pytest.mark.parametrize("shape", [(3, 16, 16, 300, 16, 16), (4, 40, 24, 700, 16, 16), (2, 17, 33, 700, 16, 32)])
def test_brute_force_tiny(oracle, shape):
    M, K, N, H, BK, BN = shape
    rng = np.random.default_rng(7)
    X, hw, dY = rng.standard_normal((M, K)), rng.standard_normal(H), rng.standard_normal((M, N))
    Y, dX, dHW = _brute(X, hw, dY, K, N, H, BK, BN, R1024, 0.5, oracle)
    for fwd, ig, wg in ((oracle.forward, oracle.input_grad, oracle.weight_grad),
                        (oracle.c_forward, oracle.c_input_grad, oracle.c_weight_grad)):
        np.testing.assert_allclose(fwd(X, hw, N, BK, BN, R1024, 0.5), Y, rtol=0, atol=1e-12)
        np.testing.assert_allclose(ig(dY, hw, K, BK, BN, R1024, 0.5), dX, rtol=0, atol=1e-12)
        np.testing.assert_allclose(wg(X, dY, H, BK, BN, R1024, 0.5), dHW, rtol=0, atol=1e-12)


@pytest.mark.parametrize("shape", [(37, 100, 150, 5000, 32, 64), (64, 128, 128, 4097, 64, 64),
                                   (20, 257, 129, 40000, 64, 32)])
def test_gradients_equal_torch_autograd_through_a_gather(oracle, shape):
    M, K, N, H, BK, BN = shape
    g = torch.Generator().manual_seed(11)
    X = torch.randn((M, K), generator=g, dtype=torch.float64, requires_grad=True)
    hw = torch.randn((H,), generator=g, dtype=torch.float64, requires_grad=True)
    dY = torch.randn((M, N), generator=g, dtype=torch.float64)
    idx = torch.from_numpy(oracle.index_map(K, N, H, BK, BN, R1024))
    Y = (X @ hw[idx]) * 1.5
    Y.backward(dY)
    x, h, d = X.detach().numpy(), hw.detach().numpy(), dY.numpy()
    for fwd, ig, wg in ((oracle.forward, oracle.input_grad, oracle.weight_grad),
                        (oracle.c_forward, oracle.c_input_grad, oracle.c_weight_grad)):
        np.testing.assert_allclose(fwd(x, h, N, BK, BN, R1024, 1.5), Y.detach().numpy(), rtol=1e-12, atol=1e-11)
        np.testing.assert_allclose(ig(d, h, K, BK, BN, R1024, 1.5), X.grad.numpy(), rtol=1e-12, atol=1e-11)
        np.testing.assert_allclose(wg(x, d, H, BK, BN, R1024, 1.5), hw.grad.numpy(), rtol=1e-12, atol=1e-11)


def test_weight_grad_invariants(oracle):
    rng = np.random.default_rng(3)
    # single tile, no collisions: the slice is the dense gradient, everything else exactly zero
    M, K, N, H, BK, BN = 9, 32, 64, 5000, 32, 64
    X, dY = rng.standard_normal((M, K)), rng.standard_normal((M, N))
    off = oracle.tile_offset(0, 0, H, BK, BN, R1024)
    for wg in (oracle.weight_grad, oracle.c_weight_grad):
        d = wg(X, dY, H, BK, BN, R1024, 2.0)
        np.testing.assert_allclose(d[off:off + BK * BN], 2.0 * (X.T @ dY).ravel(), rtol=1e-12, atol=1e-13)
        assert not d[:off].any() and not d[off + BK * BN:].any()
    # many colliding tiles: total mass is preserved (the notebooks' sum(wt_grad) == sum(grad) check)
    M, K, N, H = 8, 256, 192, 1500
    X, dY = rng.standard_normal((M, K)), rng.standard_normal((M, N))
    for wg in (oracle.weight_grad, oracle.c_weight_grad):
        d = wg(X, dY, H, 32, 32, R1024, 0.25)
        np.testing.assert_allclose(d.sum(), 0.25 * (X.T @ dY).sum(), rtol=1e-10)
    # input = identity, grad = ones: every covered slot counts how many W elements map to it
    K, N, H = 64, 64, 1100
    d = oracle.c_weight_grad(np.eye(K), np.ones((K, N)), H, 32, 32, R1024, 1.0)
    counts = np.bincount(oracle.index_map(K, N, H, 32, 32, R1024).ravel(), minlength=H)
    assert np.array_equal(d, counts.astype(np.float64)) and d.sum() == K * N


def test_linearity_and_adjointness(oracle):
    # <Y, dY> = <X, dX> = <hw, dHW> / ... : the three maps are the same bilinear form
    rng = np.random.default_rng(5)
    M, K, N, H, BK, BN = 12, 70, 90, 3000, 16, 32
    X, hw, dY = rng.standard_normal((M, K)), rng.standard_normal(H), rng.standard_normal((M, N))
    Y = oracle.c_forward(X, hw, N, BK, BN, R1024, 0.7)
    dX = oracle.c_input_grad(dY, hw, K, BK, BN, R1024, 0.7)
    dHW = oracle.c_weight_grad(X, dY, H, BK, BN, R1024, 0.7)
    s = (Y * dY).sum()
    np.testing.assert_allclose((X * dX).sum(), s, rtol=1e-11)
    np.testing.assert_allclose((hw * dHW).sum(), s, rtol=1e-11)


# ------------------------------------------------------------------ vectors made by the reference itself
def test_oracle_matches_vectors_produced_by_the_reference_kernels(oracle):
    """tests/golden/reference_vectors.npz holds inputs and outputs of the reference's own Triton
    kernels (run under Triton's CPU interpreter by tests/golden/make_reference_vectors.py).  This
    is what pins the transcription of the two-level hash, the masks and the scale."""
    d = np.load(os.path.join(GOLDEN, "reference_vectors.npz"))
    R = d["R"].tolist()
    assert R == R1024
    for name in "abc":
        M, K, N, H, BK, BN = [int(v) for v in d[name + "_shape"]]
        f = float(d[name + "_f"])
        x, hw, dy = d[name + "_x"], d[name + "_hw"], d[name + "_dy"]
        for fwd, ig, wg in ((oracle.forward, oracle.input_grad, oracle.weight_grad),
                            (oracle.c_forward, oracle.c_input_grad, oracle.c_weight_grad)):
            for ref, got in ((d[name + "_y"], fwd(x, hw, N, BK, BN, R, f)),
                             (d[name + "_dx"], ig(dy, hw, K, BK, BN, R, f)),
                             (d[name + "_dhw"], wg(x, dy, H, BK, BN, R, f))):
                assert ref.shape == got.shape
                # the reference accumulates in fp32: allow its rounding, nothing more
                assert np.abs(ref - got).max() <= 2e-6 * np.abs(got).max()


def test_oracle_against_fp16_vectors_of_the_reference_kernels(oracle):
    """tests/golden/reference_vectors_16bit.npz: the reference's kernels on fp16 tensors (Triton's
    CPU interpreter; it does not support bf16).  The float64 oracle on the same fp16 inputs must
    agree to fp16 rounding: the reference accumulates tl.dot in fp32 and rounds the output once
    (measured 2.4e-4 .. 4.0e-4), and adds the weight gradient atomically in fp16 (<= 7.6e-4)."""
    d = np.load(os.path.join(GOLDEN, "reference_vectors_16bit.npz"))
    R = d["R"].tolist()
    for name in "hi":
        assert str(d[name + "_dtype"]) == "float16"
        M, K, N, H, BK, BN = [int(v) for v in d[name + "_shape"]]
        f = float(d[name + "_f"])
        x, hw, dy = (d[name + s].astype(np.float64) for s in ("_x", "_hw", "_dy"))
        rel = lambda a, b: np.abs(a - b).max() / np.abs(b).max()
        assert rel(d[name + "_y"], oracle.forward(x, hw, N, BK, BN, R, f)) <= 1e-3
        assert rel(d[name + "_dx"], oracle.input_grad(dy, hw, K, BK, BN, R, f)) <= 1e-3
        assert rel(d[name + "_dhw"], oracle.weight_grad(x, dy, H, BK, BN, R, f)) <= 2e-3
        assert rel(d[name + "_y"], oracle.c_forward(x, hw, N, BK, BN, R, f)) <= 1e-3


# ---------------------------------------------------------------- legacy generation hash
# Row 1 of the output the reference's notebook recorded for hashed_weight = arange(1000),
# input = eye(128), a 128 x 128 layer, seed 1024 (verify.ipynb, cell 3): with an identity
# input the output is the index map itself.
NOTEBOOK_ROW1 = sum((list(range(a, a + 16)) for a in (275, 433, 591, 597, 755, 168, 326, 484)), [])
# the first numbers the legacy module printed for seed 1024 (same notebook)
NOTEBOOK_NUMBERS = [2038074743, 634329019, 1825252241, 871205357]


def test_legacy_hash_reproduces_the_notebook_row(oracle):
    R = oracle.legacy_constants(1024)
    assert R[:4] == NOTEBOOK_NUMBERS
    assert all(v % 2 == 1 for v in R[1:])
    W = oracle.materialize(np.arange(1000), 128, 128, 16, 16, R, hash_levels=3)
    assert W[1].astype(np.int64).tolist() == NOTEBOOK_ROW1
    Wc = oracle.c_materialize(np.arange(1000.0), 128, 128, 16, 16, R, hash_levels=3)
    assert np.array_equal(W, Wc)
    # identity input: forward output = W (the notebook's trick)
    assert np.array_equal(oracle.forward(np.eye(128), np.arange(1000), 128, 16, 16, R, hash_levels=3), W)


def test_legacy_hash_is_64_bit_and_uses_range_plus_one(oracle):
    R = oracle.legacy_constants(7)
    # products far beyond 2^31: Python integers vs the C restatement
    offs = oracle.c_tile_offsets(16 * 3000, 16 * 5, 70001, 16, 16, R, 3)
    for tk in (0, 1, 2999):
        for tn in range(5):
            want = ((tk * R[3] + tn * R[2] + R[1]) % R[0]) % (70001 - 256 + 1)
            assert offs[tk, tn] == want == oracle.tile_offset(tk, tn, 70001, 16, 16, R, 3)
    # H == BK*BN is legal there: every tile at offset 0
    assert not oracle.c_tile_offsets(64, 64, 256, 16, 16, R, 3).any()
    assert (oracle.c_tile_offsets(640, 640, 257, 16, 16, R, 3) <= 1).all()


@pytest.mark.parametrize("shape", [(48, 200, 136, 9000, 32, 64, 1.0), (130, 64, 64, 4097, 64, 64, 0.5),
                                   (17, 300, 77, 20000, 16, 32, 2.0)])
def test_timed_cpu_path_equals_the_oracle(oracle, shape):
    """oracle/cpu_path.py (the CPU baseline that bench.py times: gather W through the index map,
    torch.matmul, index_add_) against the numpy and C restatements, in float64 where the three
    must agree to rounding, and in its own fp32 at the fp32 tolerance."""
    import torch
    from oracle import cpu_path
    M, K, N, H, BK, BN, f = shape
    R = [45007, 29440, 22221, 32190, 14791, 1316, 35275, 26448]
    rng = np.random.default_rng(5)
    x, hw, dy = rng.standard_normal((M, K)), rng.uniform(-1, 1, H) / K ** 0.5, rng.standard_normal((M, N))
    path = cpu_path.CpuPath(K, N, H, BK, BN, R, init_factor=f)
    assert np.array_equal(path.index_map.numpy(), oracle.index_map(K, N, H, BK, BN, R))
    refs = (oracle.forward(x, hw, N, BK, BN, R, f), oracle.input_grad(dy, hw, K, BK, BN, R, f),
            oracle.weight_grad(x, dy, H, BK, BN, R, f))
    crefs = (oracle.c_forward(x, hw, N, BK, BN, R, f), oracle.c_input_grad(dy, hw, K, BK, BN, R, f),
             oracle.c_weight_grad(x, dy, H, BK, BN, R, f))
    for dt, tol in ((torch.float64, 1e-12), (torch.float32, 1e-5)):
        got = path.step(torch.from_numpy(x).to(dt), torch.from_numpy(hw).to(dt), torch.from_numpy(dy).to(dt))
        for g, r, c in zip(got, refs, crefs):
            scale = np.abs(r).max()
            assert np.abs(g.double().numpy() - r).max() <= tol * scale
            assert np.abs(g.double().numpy() - c).max() <= tol * scale
