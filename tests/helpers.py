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
