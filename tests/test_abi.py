"""CPU checks of the C ABI: the library loads, exports what include/rzlinear.h declares, the
host-side hash is bit-exact against the oracle, and bad arguments come back as status codes.
No device compute is called here."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
R1024 = [45007, 20011, 38363, 15263, 24507, 36489, 12234, 43027]
R0 = [45007, 29440, 22221, 32190, 14791, 1316, 35275, 26448]


@pytest.fixture(scope="module")
def lib():
    from rzlinear_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from rzlinear_amd import build
        build.build(verbose=False)
    return _lib.load()


def _declared():
    text = open(os.path.join(ROOT, "include", "rzlinear.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rz_[a-z_0-9]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    from rzlinear_amd import _lib
    names = _declared()
    assert sorted(_lib.EXPORTS) == names
    for n in names:
        assert hasattr(lib, n), n
    assert lib.rz_version() >= 100


def _R(r):
    return (ctypes.c_int32 * 8)(*r)


@pytest.mark.parametrize("cfg", [(1024, 1024, 65536, 64, 64), (1024, 1024, 16384, 64, 64),
                                 (2048, 2048, 16384, 64, 64), (4096, 4096, 16778, 64, 64),
                                 (512, 1024, 5243, 64, 64), (4096, 16384, 67109, 64, 64),
                                 (2048, 2048, 32768, 64, 64), (4096, 4096, 16778, 32, 64),
                                 (1000, 77, 20000, 32, 64), (99999, 99999, 66000, 256, 256),
                                 (99999, 16, 300, 16, 16)])
@pytest.mark.parametrize("levels", [1, 2])
def test_host_tile_offsets_bit_exact(lib, oracle, cfg, levels):
    from rzlinear_amd import _lib
    K, N, H, BK, BN = cfg
    for R in (R1024, R0):
        got = _lib.tile_offsets(K, N, H, BK, BN, R, levels).numpy().astype(np.int64)
        assert np.array_equal(got, oracle.c_tile_offsets(K, N, H, BK, BN, R, levels))


@pytest.mark.parametrize("cfg", [(128, 128, 1000, 16, 16), (99999, 99999, 66000, 256, 256), (99999, 16, 300, 16, 16),
                                 (40000, 500, 1000000, 16, 16), (64, 64, 256, 16, 16)])
def test_host_tile_offsets_legacy_hash(lib, oracle, cfg):
    """hash_levels = 3: the legacy generation's 64-bit hash with its prime near 2^31."""
    from rzlinear_amd import _lib
    K, N, H, BK, BN = cfg
    for seed in (1024, 7):
        R = oracle.legacy_constants(seed)
        got = _lib.tile_offsets(K, N, H, BK, BN, R, 3).numpy().astype(np.int64)
        assert np.array_equal(got, oracle.c_tile_offsets(K, N, H, BK, BN, R, 3))
    if cfg == (128, 128, 1000, 16, 16):   # tile bases behind the row the reference's notebook recorded
        R = oracle.legacy_constants(1024)
        assert _lib.tile_offsets(K, N, H, BK, BN, R, 3)[0].tolist() == [259, 417, 575, 581, 739, 152, 310, 468]


def test_status_codes(lib):
    out = (ctypes.c_int32 * 64)()
    i32p = ctypes.POINTER(ctypes.c_int32)
    call = lambda K, N, H, BK, BN, R, lv=2: lib.rz_tile_offsets(ctypes.cast(out, i32p), K, N, H, BK, BN, _R(R), lv)
    assert call(128, 128, 65536, 64, 64, R1024) == 0
    assert call(128, 128, 4096, 64, 64, R1024) == -4            # H == BK*BN
    assert call(128, 128, 100, 64, 64, R1024) == -4
    assert call(128, 128, 65536, 48, 64, R1024) == -3           # not a power of two
    assert call(128, 128, 65536, 8, 64, R1024) == -3
    assert call(128, 128, 65536, 64, 512, R1024) == -3
    assert call(0, 128, 65536, 64, 64, R1024) == -2
    assert call(128, 128, 65536, 64, 64, [2**31 - 1] + R1024[1:]) == -6
    assert call(128, 128, 65536, 64, 64, [45007, -1] + R1024[2:]) == -9
    assert call(128, 128, 65536, 64, 64, R1024, 4) == -9          # no such hash
    assert call(128, 128, 65536, 64, 64, R1024, 0) == -9
    # the legacy hash is 64-bit (no overflow status) and accepts H == BK*BN
    assert call(128, 128, 65536, 64, 64, [2**31 - 1] + R1024[1:], 3) == 0
    assert call(128, 128, 4096, 64, 64, R1024, 3) == 0
    assert call(128, 128, 4095, 64, 64, R1024, 3) == -4
    assert lib.rz_tile_offsets(None, 128, 128, 65536, 64, 64, _R(R1024), 2) == -1
    # device entry points validate before they touch the GPU
    assert lib.rz_forward(None, None, None, 1, 1, 1, 65536, 64, 64, _R(R1024), 1.0, 1, 1, 0, None) == -1
    one = ctypes.c_void_p(1)
    assert lib.rz_forward(one, one, one, 8, 128, 128, 65536, 64, 64, _R(R1024), 1.0, 128, 128, 7, None) == -5
    assert lib.rz_forward(one, one, one, 8, 128, 128, 65536, 64, 64, _R(R1024), 1.0, 64, 128, 0, None) == -2
    assert lib.rz_input_grad(one, one, one, 8, 128, 128, 4096, 64, 64, _R(R1024), 1.0, 128, 128, 0, None) == -4
    assert lib.rz_weight_grad(one, one, one, None, 0, 8, 128, 128, 65536, 64, 64, _R(R1024), 1.0, 128, 128, 1,
                              None) == -7                         # a hashed_weight beyond LDS needs a workspace
    assert lib.rz_materialize(one, one, 128, 128, 65536, 64, 64, _R(R1024), 2, 64, 0, None) == -2
    # a skinny problem splits its contraction and then needs the workspace
    need = lib.rz_forward_workspace_bytes(32, 10240, 1024, 65536, 64, 64, 0)
    assert need > 0 and need % (32 * 1024 * 4) == 0
    assert lib.rz_forward_workspace_bytes(4096, 4096, 4096, 65536, 64, 64, 1) == 0
    assert lib.rz_forward_ws(one, one, None, one, None, 0, 32, 10240, 1024, 65536, 64, 64, _R(R1024), 1.0,
                             10240, 1024, 0, None) == -7
    assert lib.rz_input_grad_ws(one, one, one, None, 0, 32, 1024, 10240, 65536, 64, 64, _R(R1024), 1.0,
                                10240, 1024, 0, None) == -7
    # a hashed_weight too large for LDS and few tiles: X^T.dY tile by tile (4 tiles of 16 KB between two margins
    # of 2 KB) and the table of tile offsets; with the fold switched off, the atomic scatter: nothing for an
    # fp32 gradient, its fp32 image for a 16-bit one
    from rzlinear_amd import _lib
    # (a 16-bit layer with a 16-bit dHW keeps the tiles in its own dtype: half the bytes; with an fp32 dHW, or told
    #  to, floats)
    assert lib.rz_weight_grad_workspace_bytes(8, 128, 128, 65536, 64, 64, 0) == 4 * 16384 + 2 * 2048 + 256
    assert lib.rz_weight_grad_workspace_bytes(8, 128, 128, 65536, 64, 64, 1) == 4 * 8192 + 2 * 2048 + 256
    assert lib.rz_weight_grad_ex_workspace_bytes(8, 128, 128, 65536, 64, 64, 1, 2, 0) == 4 * 16384 + 2 * 2048 + 256   # RZ_WG_DHW_F32
    wide = _lib.Tuning(fold_tiles=-1)
    assert lib.rz_weight_grad_hashed_workspace_bytes(8, 128, 128, 65536, 64, 64, 1, 0, 0, ctypes.byref(wide)) == 4 * 16384 + 2 * 2048 + 256
    no_fold = _lib.Tuning(fold=-1)
    assert lib.rz_weight_grad_hashed_workspace_bytes(8, 128, 128, 65536, 64, 64, 0, 0, 0, ctypes.byref(no_fold)) == 0
    assert lib.rz_weight_grad_hashed_workspace_bytes(8, 128, 128, 65536, 64, 64, 1, 0, 0, ctypes.byref(no_fold)) == 65536 * 4
    assert lib.rz_forward_hashed(one, one, None, one, None, 0, 8, 128, 128, 65536, 64, 64, _R(R1024), 5, 1.0,
                                 128, 128, 0, None, None) == -9
    # tuning overrides are validated
    bad = _lib.Tuning(tile=96)
    assert lib.rz_forward_hashed(one, one, None, one, None, 0, 8, 128, 128, 65536, 64, 64, _R(R1024), 2, 1.0,
                                 128, 128, 0, ctypes.byref(bad), None) == -9
    assert lib.rz_plan_query(0, 8, 128, 128, 65536, 64, 64, 0, 0, 0, ctypes.byref(bad), (ctypes.c_int32 * 8)()) == -9
    for code in range(0, -10, -1):
        assert lib.rz_status_string(code) not in (None, b"", b"unknown status")
    assert lib.rz_status_string(-99) == b"unknown status"


def test_tuning_overrides_of_the_cut_and_of_the_fold_tiles(lib):
    """rz_tuning.split = n asks for exactly n slices (the library's own choice where no such cut exists),
    rz_tuning.finish = -1 sends a cut to the second kernel, rz_tuning.fold_tiles = -1 keeps fp32 tiles;
    values outside their ranges are refused."""
    from rzlinear_amd import _lib
    out = (ctypes.c_int32 * 8)()
    shape = (128, 2048, 8192, 16384, 64, 64)
    for n in (2, 3, 4, 6):
        t = _lib.Tuning(tile=128, split=n)
        assert lib.rz_plan_query(0, *shape, 1, 0, 0, ctypes.byref(t), out) == 0
        assert (out[0], out[1], out[4]) == (128, n, 1)
        assert out[1] * out[2] >= 2048 and out[2] % out[3] == 0
        assert out[6] == (1 if n <= 4 else 0)          # up to four slices the kernel finishes its own tiles
        t = _lib.Tuning(tile=128, split=n, finish=-1)
        assert lib.rz_plan_query(0, *shape, 1, 0, 0, ctypes.byref(t), out) == 0 and out[6] == 0
    # a batch smaller than the tile goes to the second kernel
    t = _lib.Tuning(tile=128, split=3)
    assert lib.rz_plan_query(0, 32, 2048, 8192, 16384, 64, 64, 1, 0, 0, ctypes.byref(t), out) == 0 and (out[1], out[6]) == (3, 0)
    # 64 steps of K = 2048 cannot make 13 slices of whole steps that are all used: the library's own cut
    t = _lib.Tuning(tile=64, split=13)
    assert lib.rz_plan_query(0, 128, 2048, 8192, 16384, 64, 64, 0, 0, 0, ctypes.byref(t), out) == 0 and out[1] != 13
    for bad in (_lib.Tuning(split=17), _lib.Tuning(split=-2), _lib.Tuning(finish=1), _lib.Tuning(fold_tiles=1), _lib.Tuning(fold_tiles=-2)):
        assert lib.rz_plan_query(0, *shape, 1, 0, 0, ctypes.byref(bad), out) == -9


def test_plan_slices_begin_on_step_boundaries(lib):
    """Every slice of a cut contraction must start on a boundary of the kernel's step: a step's
    table of tile offsets assumes that the step lies inside one hashed tile or covers whole
    ones (a slice that began half-way into a 256-byte step would straddle two 128-row tiles).
    Swept over shapes, element types and forced tiles through rz_plan_query."""
    from rzlinear_amd import _lib
    rng = np.random.default_rng(2024)
    shapes = [(1024, 4352, 2048), (1024, 2176, 2048), (32, 10240, 10240), (128, 10240, 1024), (512, 8320, 1536)]
    for _ in range(300):
        shapes.append((int(rng.integers(1, 2048)), int(rng.integers(64, 12000)), int(rng.integers(64, 12000))))
    seen_cut = 0
    for (M, K, N) in shapes:
        for code in (_lib.RZ_F32, _lib.RZ_BF16):
            for tile in (0, 64, 128, 256):
                with _lib.tuning(tile=tile):
                    for op, R in ((0, K), (1, N), (2, M)):
                        q = _lib.plan_query(op, M, K, N, 1 << 20, 128, 128, code)
                        assert q["step"] in (32, 64, 128), q
                        if q["mode"] == "window":
                            continue
                        assert q["slices"] >= 1 and (q["slices"] - 1) * q["slice_len"] < R <= q["slices"] * q["slice_len"], (q, R)
                        if q["slices"] > 1:
                            seen_cut += 1
                            assert q["slice_len"] % q["step"] == 0, (M, K, N, code, tile, op, q)
    assert seen_cut > 100
    # the case that used to cut 4352 = 4 x 1088 under a 128-element step
    with _lib.tuning():
        q = _lib.plan_query(0, 1024, 4352, 2048, 1 << 20, 128, 128, _lib.RZ_BF16)
    assert q["tile"] == 128 and q["slices"] > 1 and q["slice_len"] % 128 == 0, q


def _window_geometry(H):
    """Size and number of the windows of dHW the window kernel works on: one workgroup per compute
    unit (256) while a window fits its 25600 floats of LDS, else whole rounds of 256 workgroups;
    never below 1024 floats."""
    rounds = -(-H // (25600 * 256))
    w = max((-(-H // (rounds * 256)) + 3) & ~3, 1024)
    return w, -(-H // w)


def _fold_geometry(H):
    """Restated from the comments of fold_geometry: windows of at most 32768 elements; from 128 windows on,
    whole rounds of 256; a window is a multiple of 1024 elements."""
    n = -(-H // 32768)
    if 2 * n >= 256:
        n = -(-n // 256) * 256
    w = -(-(-(-H // n)) // 1024) * 1024
    return w, -(-H // w)


def _check_fold_lists(plan, at, tiles, offsets, H, E):
    """The fold kernel's lists behind word `at` of a plan: window b's list holds exactly the tiles whose
    E elements meet [b*w, (b+1)*w), in the order in which the kernel's own search numbers tiles: pass by pass
    of 65536 tile indices, and inside a pass thread t (of 1024) holds the tiles t, t + 1024, ... of the pass.
    Returns the word behind the lists."""
    w, windows = _fold_geometry(H)
    assert (int(plan[14]), int(plan[15])) == (windows, w)
    r16 = lambda v: (v + 15) & ~15
    cap = tiles * (-(-E // w) + 1)
    list_at = r16(at + windows + 1)
    start = plan[at:at + windows + 1]
    assert start[0] == 0 and np.all(np.diff(start) >= 0) and start[-1] <= cap
    ids = np.arange(tiles)
    order = np.lexsort(((ids % 65536) // 1024, ids % 1024, ids // 65536))   # (last key first)
    total = 0
    for b in range(windows):
        meets = order[(offsets[order] < (b + 1) * w) & (offsets[order] + E > b * w)]
        assert np.array_equal(plan[list_at + start[b]:list_at + start[b + 1]], meets), b
        total += len(meets)
    assert total == start[-1] and total >= tiles
    return r16(list_at + cap)


@pytest.mark.parametrize("cfg", [(1024, 1024, 65536, 64, 64), (300, 330, 70000, 32, 64), (4096, 8192, 40000, 64, 64),
                                 (640, 640, 2000001, 64, 64), (192, 128, 7000000, 64, 64), (96, 72, 100000, 32, 64),
                                 (512, 512, 30000, 128, 128), (256, 256, 1000, 16, 16), (300, 520, 90000, 64, 32),
                                 (512, 300, 200000, 256, 128), (256, 512, 70000, 32, 256), (4800, 4800, 500000, 16, 16)])
@pytest.mark.parametrize("levels", [2, 3])
def test_layer_plan_lists_every_strip_in_every_window_it_meets(lib, oracle, cfg, levels):
    """rz_layer_plan_build against a brute-force restatement: the tile offsets are the oracle's, and
    the list of window b holds exactly the units of work of the window kernel — 32 rows by min(BN, 64)
    columns of a tile: unit s * parts + part starts at off + 32*BN*s + 64*part and spans 31*BN + min(BN, 64)
    elements — that meet [b*w, (b+1)*w), in ascending (tile, unit) order, with their offsets.  Tiles the
    window kernel does not serve (16 or 256 columns, 16 rows) get a plan with the offsets and, like every
    plan, the fold kernel's lists (_check_fold_lists)."""
    K, N, H, BK, BN = cfg
    R = R1024 if levels == 2 else oracle.legacy_constants(1024)
    nbytes = lib.rz_layer_plan_bytes(K, N, H, BK, BN)
    assert nbytes > 0 and nbytes % 64 == 0
    plan = np.zeros(nbytes // 4, dtype=np.int32)
    assert lib.rz_layer_plan_build(plan.ctypes.data, nbytes, K, N, H, BK, BN, _R(R), levels) == 0
    TK, TN = -(-K // BK), -(-N // BN)
    tiles = TK * TN
    want = oracle.c_tile_offsets(K, N, H, BK, BN, R, levels).reshape(-1)
    assert plan[0] == 0x525A4C50 and list(plan[2:9]) == [K, N, H, BK, BN, levels, tiles]
    assert np.array_equal(plan[16:16 + tiles].astype(np.int64), want)
    served = BN in (32, 64, 128) and BK in (32, 64, 128, 256)
    windows, w = int(plan[9]), int(plan[10])
    r16 = lambda v: (v + 15) & ~15
    start_at = r16(16 + tiles)
    if not served:
        assert windows == 0 and plan[11] == 0
        assert nbytes == 4 * _check_fold_lists(plan, r16(r16(start_at + 1)), tiles, want, H, BK * BN)
        return
    assert (w, windows) == _window_geometry(H)
    uc = min(BN, 64)
    parts = BN // uc
    strips, selems = (BK // 32) * parts, 31 * BN + uc
    cap = tiles * strips * (-(-selems // w) + 1)
    list_at = r16(start_at + windows + 1)
    offs_at = r16(list_at + cap)
    assert nbytes == 4 * _check_fold_lists(plan, r16(offs_at + cap), tiles, want, H, BK * BN)
    start = plan[start_at:start_at + windows + 1]
    assert start[0] == 0 and start[-1] == plan[11] and np.all(np.diff(start) >= 0) and start[-1] <= cap
    u = np.arange(strips)
    so = (want[:, None] + ((u // parts) * 32 * BN + (u % parts) * uc)[None, :]).reshape(-1)   # index = tile * units + unit
    for b in range(windows):
        meets = np.nonzero((so < (b + 1) * w) & (so + selems > b * w))[0]
        got = plan[list_at + start[b]:list_at + start[b + 1]]
        assert np.array_equal(got, meets), b
        assert np.array_equal(plan[offs_at + start[b]:offs_at + start[b + 1]], so[meets])


def test_layer_plan_argument_checks(lib):
    assert lib.rz_layer_plan_bytes(1024, 1024, 4096, 64, 64) == 0         # H must exceed the tile
    assert lib.rz_layer_plan_bytes(1024, 1024, 65536, 48, 64) == 0        # not a power of two
    n = lib.rz_layer_plan_bytes(1024, 1024, 65536, 64, 64)
    buf = np.zeros(n // 4 + 16, dtype=np.int32)
    assert lib.rz_layer_plan_build(None, n, 1024, 1024, 65536, 64, 64, _R(R1024), 2) != 0
    assert lib.rz_layer_plan_build(buf.ctypes.data, n + 64, 1024, 1024, 65536, 64, 64, _R(R1024), 2) != 0
    assert lib.rz_layer_plan_build(buf.ctypes.data, n, 1024, 1024, 65536, 64, 64, _R(R1024), 2) == 0
    # a planned call checks the plan's size against its own shape before anything is launched
    assert lib.rz_weight_grad_planned(1, 1, 1, None, None, 0, buf.ctypes.data, n - 64, 32, 1024, 1024, 65536, 64, 64,
                                      _R(R1024), 2, 1.0, 1024, 1024, 0, 0, None, None) != 0
    assert lib.rz_weight_grad_planned(1, 1, 1, None, None, 0, None, n, 32, 1024, 1024, 65536, 64, 64,
                                      _R(R1024), 2, 1.0, 1024, 1024, 0, 0, None, None) != 0
