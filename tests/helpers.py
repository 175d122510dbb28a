"""Shared pieces of the GPU parity tests: seeded inputs, tolerances, error measure."""
import numpy as np
import torch

# Stated tolerances of the hot path: normalised max error  max|out - ref| / max|ref|
#   fp32  <= 1e-4,   bf16 <= 2e-2,   fp16 <= 2e-2 (actual errors are ~1e-3).
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}

SEED_CONSTANTS = {
    1024: [45007, 20011, 38363, 15263, 24507, 36489, 12234, 43027],
    0: [45007, 29440, 22221, 32190, 14791, 1316, 35275, 26448],
}


def rel_err(out, ref):
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert out.shape == ref.shape, (out.shape, ref.shape)
    assert np.isfinite(out).all(), "non-finite values in the kernel output"
    scale = np.abs(ref).max()
    return float(np.abs(out - ref).max() / (scale if scale > 0 else 1.0))


# Element-wise bound for the 16-bit kernels, next to the normalised bound above.  The kernels
# multiply exactly (16-bit products fit fp32), accumulate in fp32 and round ONCE to the output
# type, so against the float64 oracle on the same rounded inputs every element must satisfy
#     |out - ref| <= ulp(type) * |ref|  +  1e-5 * max|ref|
# (one output rounding: 2^-8 relative for bf16, 2^-10 for fp16 covers a whole unit in the last
#  place; the second term is the fp32 accumulation over the contracted dimension).  This is
# much tighter than 2e-2 of the tensor maximum and it is what exposes a polluted edge row or
# column: the reference's own tests compare element-wise too (allclose(rtol=1e-3) in fp32,
# python/tests/test_rz_linear.py:73,:113,:141).
ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -22}
# Largest relative error of ONE rounding to nearest: half a unit in the last place of a significand of 8 (bf16)
# or 11 (fp16) bits.
ROUNDING = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}


def elementwise_excess(out, ref, dtype, floor=1e-5, slack=None):
    """Largest |out - ref| / (ulp*|ref| + floor*max|ref| + slack) over all elements: <= 1 passes."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert out.shape == ref.shape, (out.shape, ref.shape)
    assert np.isfinite(out).all(), "non-finite values in the kernel output"
    scale = np.abs(ref).max()
    bound = ULP[dtype] * np.abs(ref) + floor * (scale if scale > 0 else 1.0)
    if slack is not None:
        bound = bound + slack
    return float((np.abs(out - ref) / bound).max()) if out.size else 0.0


def stored_tiles_slack(oracle, x64, dy64, shape, R, scale, dtype, hash_levels=None):
    """What the element-wise bound of a 16-bit dHW gains when the weight gradient goes through the fold with
    the tiles of X^T.dY stored in the layer's dtype (rz_tuning.fold_tiles = 0): every stored value — one per
    element of X^T.dY and slice of M, complete fp32 sums — is rounded once (ROUNDING[dtype] of its magnitude
    at most) before the fold adds the values of a slot up in fp32.  Returns the allowance per element of dHW, or None
    where no plan of this problem takes that path (fp32 layers; LDS image, window kernel, atomics)."""
    from rzlinear_amd import _lib
    if dtype == torch.float32:
        return None
    M, K, N, H, BK, BN = shape
    code = _lib.RZ_BF16 if dtype == torch.bfloat16 else _lib.RZ_F16
    plans = [_lib.plan_query(2, M, K, N, H, BK, BN, code, planned=p) for p in (False, True)]
    folds = [p for p in plans if p["mode"] == "fold"]
    if not folds:
        return None
    idx = oracle.index_map(K, N, H, BK, BN, R) if hash_levels is None else oracle.index_map(K, N, H, BK, BN, R, hash_levels)
    slack = np.zeros((H,), dtype=np.float64)
    for p in folds:
        step = p["slice_len"] if p["slices"] > 1 else M
        stored = sum(np.abs(x64[m:m + step].T @ dy64[m:m + step]) for m in range(0, M, step)) * abs(scale)
        s = np.zeros((H,), dtype=np.float64)
        np.add.at(s, idx.reshape(-1), stored.reshape(-1))
        slack = np.maximum(slack, s)
    return ROUNDING[dtype] * slack


def assert_close(out, ref, dtype, what="", slack=None):
    """Both bounds: the stated normalised tolerance and, element by element, the rounding bound
    (plus `slack`, an allowance per element, where a path rounds more than once: see stored_tiles_slack)."""
    e = rel_err(out, ref)
    assert e <= TOL[dtype], "%s: normalised max error %.3g > %.3g" % (what, e, TOL[dtype])
    x = elementwise_excess(out, ref, dtype, slack=slack)
    if x > 1.0:
        out = np.asarray(out, dtype=np.float64)
        ref = np.asarray(ref, dtype=np.float64)
        scale = np.abs(ref).max()
        bad = np.abs(out - ref) / (ULP[dtype] * np.abs(ref) + 1e-5 * (scale if scale > 0 else 1.0) + (0.0 if slack is None else slack))
        at = np.unravel_index(int(bad.argmax()), bad.shape)
        raise AssertionError("%s: element %s is %.6g, expected %.6g (%.2f x the element-wise bound; %d elements "
                             "beyond it)" % (what, at, out[at], ref[at], x, int((bad > 1.0).sum())))


def make_inputs(M, K, N, H, dtype, seed, device="cuda"):
    """X ~ N(0,1), hashed_weight ~ U(-1/sqrt(K), 1/sqrt(K)), dY ~ N(0,1), rounded to dtype.
    Returns the device tensors and their exact float64 images for the oracle."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((M, K), generator=g).to(dtype)
    hw = ((torch.rand((H,), generator=g) * 2 - 1) / K ** 0.5).to(dtype)
    dy = torch.randn((M, N), generator=g).to(dtype)
    f64 = lambda t: t.to(torch.float64).numpy()
    return (x.to(device), hw.to(device), dy.to(device)), (f64(x), f64(hw), f64(dy))


def rargs(R):
    """R7..R0 in the positional order of the launchers."""
    return (R[7], R[6], R[5], R[4], R[3], R[2], R[1], R[0])
