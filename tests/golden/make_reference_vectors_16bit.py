"""Writes tests/golden/reference_vectors_16bit.npz: the REFERENCE's forward, input-grad and
weight-grad launchers on small fp16 and bf16 CPU tensors, run under Triton's CPU interpreter
(TRITON_INTERPRET=1) in the build container, like make_reference_vectors.py does for fp32.

Why: how the reference's kernels behave on 16-bit tensors (fp32 accumulation of tl.dot, one
rounding of the output, atomic adds in the tensor's own type for the weight gradient) is
pinned by nothing the reference ships.  Only the vectors (data) are committed.

    python tests/golden/make_reference_vectors_16bit.py [/root/reference/python]
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
    # name, dtype, M, K, N, H, BLOCK_SIZE_M, BLOCK_SIZE_K, BLOCK_SIZE_N, init_factor
    ("h", torch.float16, 32, 64, 128, 5000, 32, 32, 64, 1.0),
    ("i", torch.float16, 48, 96, 80, 3000, 16, 32, 16, 0.5),       # ragged: masks on M, K and N
    ("j", torch.bfloat16, 32, 64, 128, 5000, 32, 32, 64, 1.0),
    ("k", torch.bfloat16, 48, 96, 80, 3000, 16, 32, 16, 0.5),
]
out = {"R": np.array(R, dtype=np.int32)}
for name, dtype, M, K, N, H, BM, BK, BN, f in CASES:
    g = torch.Generator().manual_seed(200 + len(out))
    x = torch.randn((M, K), generator=g).to(dtype)
    hw = (torch.randn((H,), generator=g) / 8).to(dtype)
    dy = torch.randn((M, N), generator=g).to(dtype)
    consts = (R[7], R[6], R[5], R[4], R[3], R[2], R[1], R[0])
    kw = dict(allow_tf32=False, allow_autotune=False, BLOCK_SIZE_M=BM, BLOCK_SIZE_N=BN, BLOCK_SIZE_K=BK)
    try:
        y = rz_linear_forward_tl(x, hw, f, M, K, N, H, *consts, GROUP_SIZE=4, **kw)
        dx = rz_linear_backward_input_grad_tl(dy, hw, f, M, K, N, H, *consts, GROUP_SIZE=4, **kw)
        dhw = rz_linear_backward_weight_grad_tl(x, dy, f, M, K, N, H, *consts, GROUP_SIZE=8, **kw)
    except Exception as e:   # the interpreter may not support a type: say so and go on
        print(name, str(dtype), "not produced:", type(e).__name__, str(e)[:200])
        continue
    f32 = lambda t: t.float().numpy()
    out.update({name + "_shape": np.array([M, K, N, H, BK, BN], dtype=np.int64), name + "_f": np.float64(f),
                name + "_dtype": np.array(str(dtype).split(".")[-1]),
                name + "_x": f32(x), name + "_hw": f32(hw), name + "_dy": f32(dy),
                name + "_y": f32(y), name + "_dx": f32(dx), name + "_dhw": f32(dhw)})
    print(name, str(dtype), "ok", y.dtype, dx.dtype, dhw.dtype, float(y.float().abs().max()))
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors_16bit.npz")
np.savez_compressed(path, **out)
print("wrote", path, os.path.getsize(path), "bytes")
