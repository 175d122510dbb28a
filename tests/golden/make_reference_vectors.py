"""Writes tests/golden/reference_vectors.npz: inputs and outputs of the REFERENCE's own forward,
input-grad and weight-grad launchers on small CPU tensors, produced by running the reference's
Triton kernels under Triton's CPU interpreter (TRITON_INTERPRET=1) in the build container.

Why: the two-level tile hash lives only inside those kernels (python/rz_linear/impl/
RzLinearForward.py:316, RzLinearBackward.py:369,:686,:716); the reference ships no test or
fixture that pins it, so nothing but an execution can confirm that the oracle transcribed it
correctly.  Only the vectors (data) are committed; the reference source is not copied and is
not needed to run the tests.

    python tests/golden/make_reference_vectors.py [/root/reference/python]
"""
import os
import sys

os.environ["TRITON_INTERPRET"] = "1"

import numpy as np
import torch

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/python"
sys.path.insert(0, ref)

from rz_linear.impl.RzLinearForward import rz_linear_forward_tl          # noqa: E402
from rz_linear.impl.RzLinearBackward import (rz_linear_backward_input_grad_tl,   # noqa: E402
                                             rz_linear_backward_weight_grad_tl)

R = [45007, 20011, 38363, 15263, 24507, 36489, 12234, 43027]       # seed 1024, index = subscript
CASES = [
    # name, M, K, N, H, BLOCK_SIZE_M, BLOCK_SIZE_K, BLOCK_SIZE_N, init_factor
    ("a", 32, 64, 128, 5000, 32, 32, 64, 1.0),
    ("b", 48, 96, 80, 3000, 16, 32, 16, 0.5),        # ragged: masks on M, K and N
    ("c", 16, 128, 64, 4200, 16, 64, 64, 2.0),
]
out = {"R": np.array(R, dtype=np.int32)}
for name, M, K, N, H, BM, BK, BN, f in CASES:
    g = torch.Generator().manual_seed(100 + len(out))
    x = torch.randn((M, K), generator=g)
    hw = torch.randn((H,), generator=g)
    dy = torch.randn((M, N), generator=g)
    consts = (R[7], R[6], R[5], R[4], R[3], R[2], R[1], R[0])
    kw = dict(allow_tf32=False, allow_autotune=False, BLOCK_SIZE_M=BM, BLOCK_SIZE_N=BN, BLOCK_SIZE_K=BK)
    y = rz_linear_forward_tl(x, hw, f, M, K, N, H, *consts, GROUP_SIZE=4, **kw)
    dx = rz_linear_backward_input_grad_tl(dy, hw, f, M, K, N, H, *consts, GROUP_SIZE=4, **kw)
    dhw = rz_linear_backward_weight_grad_tl(x, dy, f, M, K, N, H, *consts, GROUP_SIZE=8, **kw)
    out.update({name + "_shape": np.array([M, K, N, H, BK, BN], dtype=np.int64), name + "_f": np.float64(f),
                name + "_x": x.numpy(), name + "_hw": hw.numpy(), name + "_dy": dy.numpy(),
                name + "_y": y.numpy(), name + "_dx": dx.numpy(), name + "_dhw": dhw.numpy()})
    print(name, "ok", y.shape, dx.shape, dhw.shape, float(y.abs().max()))
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")
np.savez_compressed(path, **out)
print("wrote", path, os.path.getsize(path), "bytes")
