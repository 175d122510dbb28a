"""The fold kernel's division of a window's tiles among the workgroups that share the window
(rzlinear_amd/csrc/rz_fold.h), restated on the CPU.

The kernel numbers the tiles that land in a window in an order that depends on the table of tile
offsets alone — pass by pass of 64 * 1024 tile indices; inside a pass thread by thread (thread t
holds the indices lo + t + 1024 j), and inside a thread by ascending j — and share s of S takes the
numbers [s * all / S, (s + 1) * all / S), in chunks of as many tiles as its list holds.  What this
file checks is the property the scheme exists for: whatever the offsets, the shares' tiles are a
partition of the window's tiles, also when a share needs several chunks (the case in which an
earlier scheme, which cut the index range in halves per share, took tiles twice or not at all).
The GPU test of the same case is tests/test_gpu_weight_grad_ex.py."""
import numpy as np
import pytest

SCAN, THREADS, LIST = 64, 1024, 2048


def window_tiles(offsets, w0, wlen, E):
    rel = offsets.astype(np.int64) - w0
    return np.nonzero((rel > -E) & (rel < wlen))[0]


def numbered(offsets, w0, wlen, E):
    """Tile ids of the window in the kernel's numbering."""
    order = []
    n = len(offsets)
    for lo in range(0, n, SCAN * THREADS):
        span = min(SCAN * THREADS, n - lo)
        ids = window_tiles(offsets[lo:lo + span], w0, wlen, E)
        t, j = ids % THREADS, ids // THREADS
        order.extend((lo + ids[np.lexsort((j, t))]).tolist())   # thread-major, then the thread's bits
    return order


def share_chunks(order, share, shares, per_tile):
    """The chunks (pass, list of tile ids) that one share works through, in order."""
    n = len(order)
    lo, hi = share * n // shares, (share + 1) * n // shares
    cap = LIST // per_tile
    chunks = []
    # (per pass, as the kernel does it; the passes are recovered from the ids)
    passes = {}
    for rank, tid in enumerate(order):
        passes.setdefault(tid // (SCAN * THREADS), []).append((rank, tid))
    for k in sorted(passes):
        ranks = passes[k]
        want_lo, want_hi = max(lo, ranks[0][0]), min(hi, ranks[-1][0] + 1)
        for c in range(want_lo, want_hi, cap):
            chunks.append((k, [tid for rank, tid in ranks if c <= rank < min(c + cap, want_hi)]))
    return chunks


@pytest.mark.parametrize("tiles,H,E,shares,per_tile", [
    (589824, 500000, 256, 16, 1),      # K = N = 12288, 16 x 16 tiles: lists overflow in every share
    (200000, 150000, 4096, 4, 2),      # tiles of two runs
    (70000, 40000, 256, 128, 8),       # eight slices: a list holds 256 tiles
    (5000, 100000, 1024, 7, 1),        # no overflow, odd number of shares
    (131073, 33000, 256, 3, 1),        # a last pass of one tile
])
def test_shares_partition_the_tiles_of_every_window(tiles, H, E, shares, per_tile):
    rng = np.random.default_rng(tiles + shares)
    offsets = rng.integers(0, H - E, size=tiles).astype(np.int32)
    window = -(-H // max(1, -(-H // 32768)))
    window = -(-window // THREADS) * THREADS
    overflowed = False
    for w0 in range(0, H, window):
        wlen = min(window, H - w0)
        order = numbered(offsets, w0, wlen, E)
        expect = sorted(window_tiles(offsets, w0, wlen, E).tolist())
        taken = []
        for s in range(shares):
            chunks = share_chunks(order, s, shares, per_tile)
            assert all(0 < len(c) * per_tile <= LIST for _, c in chunks)
            overflowed |= len({k for k, _ in chunks}) < len(chunks)     # two chunks in one pass
            taken.extend(t for _, c in chunks for t in c)
        assert sorted(taken) == expect          # every tile of the window exactly once
    if (tiles, shares) == (589824, 16):
        assert overflowed
