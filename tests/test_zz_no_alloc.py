"""rz_weight_grad_static: the weight gradient through the library's own static device scratch
(no workspace argument, no allocation), against rz_weight_grad with a caller-owned workspace
and against the oracle.  Two calls in a row on the same GPU, the second on a smaller problem, so
that whatever the first call left in the shared scratch array must not leak into the second."""
import ctypes
import sys

import numpy as np
import pytest
import torch

from helpers import SEED_CONSTANTS, TOL, assert_close, make_inputs, rel_err, stored_tiles_slack

pytestmark = pytest.mark.gpu

R1024 = SEED_CONSTANTS[1024]
SCRATCH_BYTES = 32 << 20


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _both(lib, shape, dtype, seed, oracle):
    """dHW of one problem through both entry points; returns (static, workspace, oracle, whether
    the workspace the plan asks for fits the static scratch: if not, the static entry point takes
    the atomic scatter instead)."""
    from rzlinear_amd import _lib
    M, K, N, H, BK, BN = shape
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, dtype, seed=seed)
    code = _lib.dtype_code(x)
    R = (ctypes.c_int32 * 8)(*R1024)
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.rz_weight_grad_workspace_bytes(M, K, N, H, BK, BN, code)
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device="cuda")
    # poison the outputs: both entry points overwrite dHW completely
    a = torch.full((H,), float("nan"), dtype=dtype, device="cuda")
    b = torch.full((H,), float("nan"), dtype=dtype, device="cuda")
    _lib.check(lib.rz_weight_grad_static(x.data_ptr(), dy.data_ptr(), a.data_ptr(), M, K, N, H, BK, BN, R, 0.5,
                                         K, N, code, stream))
    _lib.check(lib.rz_weight_grad(x.data_ptr(), dy.data_ptr(), b.data_ptr(), ws.data_ptr(), need, M, K, N, H,
                                  BK, BN, R, 0.5, K, N, code, stream))
    torch.cuda.synchronize()
    slack = stored_tiles_slack(oracle, x64, dy64, shape, R1024, 0.5, dtype)
    return a, b, oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5), need <= SCRATCH_BYTES, slack


# (first problem, smaller second problem, how the plan carries the first one out in bf16)
PAIRS = [
    ((768, 512, 640, 9000, 64, 64), (200, 256, 192, 5000, 64, 64), "lds_image"),
    ((512, 384, 512, 70000, 64, 64), (96, 128, 192, 40000, 32, 64), "fold"),
    ((512, 512, 768, 200000, 256, 256), (96, 256, 256, 100000, 256, 128), "atomics"),   # tiles too large to fold
    ((32, 4096, 8192, 1 << 21, 64, 64), (16, 4096, 8192, 1 << 21, 64, 64), "window"),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("pair", PAIRS, ids=lambda p: p[2])
def test_static_scratch_matches_the_workspace_entry_point(oracle, pair, dtype):
    from rzlinear_amd import _lib
    lib = _lib.load()
    first, second, mode = pair
    for i, shape in enumerate((first, second)):
        M, K, N, H, BK, BN = shape
        plan = _lib.plan_query(2, M, K, N, H, BK, BN, _lib.RZ_BF16 if dtype == torch.bfloat16 else _lib.RZ_F32)
        _say("static scratch", mode, "call", i, shape, dtype, plan)
        if dtype == torch.bfloat16 and i == 0:
            assert plan["mode"] == mode, plan      # the scratch layouts are all exercised
        a, b, ref, fits, slack = _both(lib, shape, dtype, seed=50 + i, oracle=oracle)
        assert fits or dtype != torch.bfloat16   # (the bf16 pairs exercise the scratch layouts named above)
        f = lambda t: t.float().cpu().numpy()
        if plan["mode"] == "atomics" or not fits:
            # global atomics: the summation order is not fixed, compare within the tolerance
            assert rel_err(f(a), f(b).astype(np.float64)) <= TOL[dtype]
        else:
            assert torch.equal(a, b)            # fixed summation order: the same bits
        assert_close(f(a), ref, dtype, "dHW (static scratch)", slack=slack)
        assert_close(f(b), ref, dtype, "dHW (workspace)", slack=slack)


def test_static_scratch_gives_up_the_fold_when_its_buffer_does_not_fit(oracle):
    """rz_weight_grad stores X^T.dY tile by tile for this problem (4*K*N bytes and more); the
    static entry point cannot, and takes the scatter kernel instead of refusing."""
    from rzlinear_amd import _lib
    lib = _lib.load()
    M, K, N, H, BK, BN = 40, 4096, 8192, 200000, 64, 64
    assert _lib.plan_query(2, M, K, N, H, BK, BN, _lib.RZ_BF16)["mode"] == "fold"
    assert lib.rz_weight_grad_workspace_bytes(M, K, N, H, BK, BN, _lib.RZ_BF16) > SCRATCH_BYTES
    _say("static scratch, fold does not fit", (M, K, N, H))
    (x, _, dy), (x64, _, dy64) = make_inputs(M, K, N, H, torch.bfloat16, seed=71)
    R = (ctypes.c_int32 * 8)(*R1024)
    a = torch.full((H,), float("nan"), dtype=torch.bfloat16, device="cuda")
    _lib.check(lib.rz_weight_grad_static(x.data_ptr(), dy.data_ptr(), a.data_ptr(), M, K, N, H, BK, BN, R, 0.5,
                                         K, N, _lib.RZ_BF16, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert_close(a.float().cpu().numpy(), oracle.weight_grad(x64, dy64, H, BK, BN, R1024, 0.5), torch.bfloat16,
                 "dHW (static scratch, scatter instead of fold)")


def test_static_scratch_refuses_what_does_not_fit():
    from rzlinear_amd import _lib
    lib = _lib.load()
    M, K, N, H = 8192, 8192, 8192, 30000
    assert lib.rz_weight_grad_workspace_bytes(M, K, N, H, 64, 64, _lib.RZ_BF16) > SCRATCH_BYTES
    one = ctypes.c_void_p(256)
    R = (ctypes.c_int32 * 8)(*R1024)
    st = lib.rz_weight_grad_static(one, one, one, M, K, N, H, 64, 64, R, 1.0, K, N, _lib.RZ_BF16, None)
    assert st == -10 and b"32 MiB" in lib.rz_status_string(st)
    # argument errors come back as from rz_weight_grad
    assert lib.rz_weight_grad_static(None, one, one, 64, 64, 64, 5000, 64, 64, R, 1.0, 64, 64, 0, None) == -1
    assert lib.rz_weight_grad_static(one, one, one, 64, 64, 64, 4096, 64, 64, R, 1.0, 64, 64, 0, None) == -4


def test_static_scratch_is_that_of_the_device_that_holds_the_gradient():
    """The scratch array used is the current device's; a dHW that is not memory of that device (here:
    host memory) would make the kernels work in another address space, and is refused."""
    from rzlinear_amd import _lib
    lib = _lib.load()
    M, K, N, H = 64, 64, 64, 5000
    x = torch.zeros((M, K), device="cuda")
    dy = torch.zeros((M, N), device="cuda")
    host = torch.zeros((H,))
    R = (ctypes.c_int32 * 8)(*R1024)
    st = lib.rz_weight_grad_static(x.data_ptr(), dy.data_ptr(), host.data_ptr(), M, K, N, H, 64, 64, R, 1.0, K, N,
                                   _lib.RZ_F32, torch.cuda.current_stream().cuda_stream)
    assert st == -9
    dev = torch.zeros((H,), device="cuda")
    _lib.check(lib.rz_weight_grad_static(x.data_ptr(), dy.data_ptr(), dev.data_ptr(), M, K, N, H, 64, 64, R, 1.0, K, N,
                                         _lib.RZ_F32, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
