"""Ragged shapes: the kernels keep their direct global-to-LDS staging (16-bit: the tiles of 128 and
256; fp32: every tile), fetch edge pieces from inside the operands and clear the excess of a
partial last contraction step in LDS.  Checked against the CPU oracle for every op and tile, with
and without the bias-gradient column sums."""
import sys

import pytest
import torch

from helpers import SEED_CONSTANTS, TOL, assert_close, make_inputs, rargs, rel_err, stored_tiles_slack

pytestmark = pytest.mark.gpu

R1024 = SEED_CONSTANTS[1024]

# (M, K, N, H, BK, BN)
CASES = [
    (1000, 512, 1000, 9000, 64, 64),     # forward contracts K = 8 steps; M, N ragged
    (1000, 1000, 512, 9000, 64, 64),     # input-grad contracts N
    (1024, 1000, 520, 9000, 64, 64),     # weight-grad contracts M; K, N multiples of 8 only
    (320, 136, 264, 70000, 32, 64),      # one ragged tile each way, atomic scatter
    (640, 1001, 520, 9000, 64, 64),      # K not a multiple of 8: weight-grad must use the checked kernel
    (129, 128, 129, 3000, 16, 16),       # a single row / column beyond a tile
    (1000, 512, 520, 9000, 64, 64),      # weight-grad: the last of 16 R steps holds 40 rows
    (70, 256, 256, 9000, 64, 64),        # two R steps, the second with 6 rows
    (40, 256, 384, 9000, 64, 64),        # a single, partial R step
    (4100, 192, 160, 30000, 64, 64),     # sliced M: only the last slice ends in a partial step
    (65, 1024, 1024, 200000, 64, 64),    # one row into the second step, atomic scatter
    (300, 72, 200, 9000, 16, 16),        # forward: one complete R step and one piece of the next
    (256, 8, 136, 3000, 16, 16),         # forward: a single R step holding one piece
    (200, 264, 8, 3000, 32, 64),         # input-grad: the same
]
_id = lambda s: "x".join(map(str, s))


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


FORMS = [(128, torch.bfloat16), (256, torch.bfloat16), (128, torch.float16), (256, torch.float16),
         (32, torch.float32), (64, torch.float32), (128, torch.float32), (256, torch.float32)]


@pytest.mark.parametrize("form", FORMS, ids=lambda f: "%d-%s" % (f[0], str(f[1]).split(".")[-1]))
@pytest.mark.parametrize("shape", CASES, ids=_id)
def test_ragged_edges_with_direct_staging(oracle, tuned, shape, form):
    tile, dtype = form
    from rzlinear_amd.impl.RzLinearBackward import (rz_linear_backward_input_grad_tl,
                                                    rz_linear_backward_weight_bias_grad_tl,
                                                    rz_linear_backward_weight_grad_tl)
    from rzlinear_amd.impl.RzLinearForward import rz_linear_forward_bias_tl
    from rzlinear_amd import _lib
    tuned(tile=tile)
    M, K, N, H, BK, BN = shape
    _say("ragged direct", shape, tile, dtype)
    (x, hw, dy), (x64, hw64, dy64) = make_inputs(M, K, N, H, dtype, seed=41)
    bias = torch.linspace(-1, 1, N).to(dtype).cuda()
    kw = dict(BLOCK_SIZE_K=BK, BLOCK_SIZE_N=BN)
    y = rz_linear_forward_bias_tl(x, hw, bias, 1.0, M, K, N, H, *rargs(R1024), **kw)
    dx = rz_linear_backward_input_grad_tl(dy, hw, 1.0, M, K, N, H, *rargs(R1024), **kw)
    dhw = rz_linear_backward_weight_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), **kw)
    dhw2, dbias = rz_linear_backward_weight_bias_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), **kw)
    torch.cuda.synchronize()
    f = lambda t: t.float().cpu().numpy()
    # element by element (one output rounding + fp32 accumulation), not only against the tensor
    # maximum: a polluted edge row or column must not hide behind large elements elsewhere
    assert_close(f(y), oracle.forward(x64, hw64, N, BK, BN, R1024) + bias.double().cpu().numpy(), dtype, "Y")
    assert_close(f(dx), oracle.input_grad(dy64, hw64, K, BK, BN, R1024), dtype, "dX")
    ref = oracle.weight_grad(x64, dy64, H, BK, BN, R1024)
    with _lib.tuning(tile=tile):
        slack = stored_tiles_slack(oracle, x64, dy64, shape, R1024, 1.0, dtype)
    assert_close(f(dhw), ref, dtype, "dHW", slack=slack)
    assert_close(f(dhw2), ref, dtype, "dHW (with bias gradient)", slack=slack)
    assert_close(f(dbias), dy64.sum(axis=0), dtype, "dbias")
    # the bounds-checked kernels give the same results
    tuned(tile=tile, clamp=-1)
    y2 = rz_linear_forward_bias_tl(x, hw, bias, 1.0, M, K, N, H, *rargs(R1024), **kw)
    dx2 = rz_linear_backward_input_grad_tl(dy, hw, 1.0, M, K, N, H, *rargs(R1024), **kw)
    torch.cuda.synchronize()
    dhw3, dbias3 = rz_linear_backward_weight_bias_grad_tl(x, dy, 1.0, M, K, N, H, *rargs(R1024), **kw)
    torch.cuda.synchronize()
    if dtype == torch.float32:
        # (the directly staged fp32 kernels pair the elements of a contraction step differently: same sums, another order)
        assert_close(f(y2), oracle.forward(x64, hw64, N, BK, BN, R1024) + bias.double().cpu().numpy(), dtype, "Y (bounds-checked)")
        assert_close(f(dx2), oracle.input_grad(dy64, hw64, K, BK, BN, R1024), dtype, "dX (bounds-checked)")
    else:
        assert torch.equal(y, y2) and torch.equal(dx, dx2)
    assert_close(f(dhw3), ref, dtype, "dHW (bounds-checked)", slack=slack)
    assert_close(f(dbias3), dy64.sum(axis=0), dtype, "dbias (bounds-checked)")
