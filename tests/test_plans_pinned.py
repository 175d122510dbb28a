"""The plan the library takes for every baseline configuration and for the reference's benchmark grid,
pinned: C tile, slices of the contracted dimension and the way the weight gradient reaches dHW, for
forward / input-grad / weight-grad.  The planner (rzlinear_amd/csrc/rz_launch.h) is a model fitted to
measurements; refitting it for one shape must not silently move another.  A deliberate change of plan
updates this table — together with the measurement that justifies it."""
import pytest

from rzlinear_amd import _lib

F32, BF16, F16 = _lib.RZ_F32, _lib.RZ_BF16, _lib.RZ_F16

# name: ((M, K, N, H, BLOCK_K, BLOCK_N, dtype), [(tile, slices, mode) for forward, input-grad, weight-grad])
# (tile 32 = the 32 x 64 C tile of the fp32 kernels; 0 = the window kernel, which has no C tile)
PLANS = {
    "cpu_ref_1024 fp32": ((1024, 1024, 1024, 65536, 64, 64, F32), [(64, 1, "store"), (64, 1, "store"), (64, 1, "fold")]),
    "square1024 fp32": ((1024, 1024, 1024, 16384, 64, 64, F32), [(64, 1, "store"), (64, 1, "store"), (128, 4, "lds_image")]),
    "square1024 bf16": ((1024, 1024, 1024, 16384, 64, 64, BF16), [(64, 1, "store"), (64, 1, "store"), (128, 4, "lds_image")]),
    "square2048 fp32": ((2048, 2048, 2048, 16384, 64, 64, F32), [(128, 1, "store"), (128, 1, "store"), (256, 4, "lds_image")]),
    "square2048 bf16": ((2048, 2048, 2048, 16384, 64, 64, BF16), [(128, 1, "store"), (128, 1, "store"), (128, 1, "lds_image")]),
    "square4096 fp32": ((4096, 4096, 4096, 16778, 64, 64, F32), [(256, 1, "store"), (256, 1, "store"), (256, 1, "lds_image")]),
    "square4096 bf16": ((4096, 4096, 4096, 16778, 64, 64, BF16), [(256, 1, "store"), (256, 1, "store"), (256, 1, "lds_image")]),
    "square4096 fp16": ((4096, 4096, 4096, 16778, 64, 64, F16), [(256, 1, "store"), (256, 1, "store"), (256, 1, "lds_image")]),
    "rec_mlp bf16": ((16384, 512, 1024, 5243, 64, 64, BF16), [(256, 1, "store"), (128, 1, "store"), (128, 8, "lds_image")]),
    "ffn bf16": ((8192, 4096, 16384, 67109, 64, 64, BF16), [(256, 1, "store"), (256, 1, "store"), (256, 1, "fold")]),
    "collision fp32": ((32768, 2048, 2048, 32768, 64, 64, F32), [(256, 1, "store"), (256, 1, "store"), (256, 4, "lds_image")]),
    "grid_32_1024 fp32": ((32, 1024, 1024, 65536, 32, 64, F32), [(32, 6, "split"), (32, 6, "split"), (64, 1, "fold")]),
    "grid_32_1024 bf16": ((32, 1024, 1024, 65536, 32, 64, BF16), [(64, 1, "store"), (64, 1, "store"), (64, 1, "fold")]),
    "grid_32_10240 fp32": ((32, 10240, 10240, 6553600, 32, 64, F32), [(32, 3, "split"), (32, 3, "split"), (0, 1, "window")]),
    "grid_32_10240 bf16": ((32, 10240, 10240, 6553600, 32, 64, BF16), [(128, 3, "split"), (128, 3, "split"), (0, 1, "window")]),
    "grid_128_1024 fp32": ((128, 1024, 1024, 65536, 32, 64, F32), [(64, 6, "split"), (64, 6, "split"), (64, 1, "fold")]),
    "grid_128_1024 bf16": ((128, 1024, 1024, 65536, 32, 64, BF16), [(64, 1, "store"), (64, 1, "store"), (64, 1, "fold")]),
    "grid_128_10240 fp32": ((128, 10240, 10240, 6553600, 32, 64, F32), [(128, 3, "split"), (128, 3, "split"), (0, 1, "window")]),
    "grid_128_10240 bf16": ((128, 10240, 10240, 6553600, 32, 64, BF16), [(128, 3, "split"), (128, 3, "split"), (0, 1, "window")]),
    "grid_1024_1024 fp32": ((1024, 1024, 1024, 65536, 32, 64, F32), [(64, 1, "store"), (64, 1, "store"), (64, 1, "fold")]),
    "grid_1024_1024 bf16": ((1024, 1024, 1024, 65536, 32, 64, BF16), [(64, 1, "store"), (64, 1, "store"), (64, 1, "fold")]),
    "grid_1024_10240 fp32": ((1024, 10240, 10240, 6553600, 32, 64, F32), [(64, 1, "store"), (64, 1, "store"), (128, 1, "fold")]),
    "grid_1024_10240 bf16": ((1024, 10240, 10240, 6553600, 32, 64, BF16), [(256, 3, "split"), (256, 3, "split"), (256, 1, "fold")]),
}


@pytest.mark.parametrize("name", sorted(PLANS))
def test_plan_of_a_baseline_configuration_is_what_was_measured(name):
    (M, K, N, H, BK, BN, code), want = PLANS[name]
    got = []
    for op in (0, 1, 2):
        q = _lib.plan_query(op, M, K, N, H, BK, BN, code, planned=True)   # (as the launchers ask: with a layer plan)
        got.append((q["tile"], q["slices"], q["mode"]))
    assert got == want


def test_no_baseline_configuration_takes_the_atomic_scatter():
    """Global atomics — the one path that leaves the order of the additions open — serve none of the
    configurations above; the library keeps them for hashed tiles too large to fold (more than 16384
    elements) and for many small tiles under a batch of a few rows, where they are faster."""
    assert all(mode != "atomics" for _, plan in PLANS.values() for _, _, mode in plan)
    assert _lib.plan_query(2, 128, 2048, 1024, 1 << 20, 256, 128, BF16)["mode"] == "atomics"
