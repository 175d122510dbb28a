"""CPU oracle of the RzLinear hot path — TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the CPU-baseline leg of the benchmark may import this
module; the product package never does.  Two independent restatements live here:

  * ``Numpy``-level functions (``tile_offsets``, ``index_map``, ``materialize``, ``forward``,
    ``input_grad``, ``weight_grad``): the design of the reference's own tests — build the
    dense W by gathering tiles, then use a library matmul; reduce the dense weight gradient
    into hashed_weight by a scatter-add (python/tests/test_rz_linear.py:21-33,:77-90), with
    the two-level hash of the kernels (python/rz_linear/impl/RzLinearForward.py:316).
    Everything is float64.
  * ``c_*`` functions: ctypes calls into oracle/librz_oracle.so (rz_oracle.c), which follows
    the loop structure of the device kernels instead.

Parity status: pinned.  The reference holds no golden vectors for the two-level hash, so they
were produced once by running its own Triton kernels under Triton's CPU interpreter
(tests/golden/make_reference_vectors.py -> tests/golden/reference_vectors.npz); both
restatements agree with them to fp32 rounding (and with fp16 vectors made the same way,
tests/golden/reference_vectors_16bit.npz, to fp16 rounding), and tests/test_oracle.py adds
known-answer and invariant tests and checks the two restatements against each other.  The
reference's bf16 behaviour is unpinned: the interpreter does not run bf16.
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "librz_oracle.so")

# hash constants [R0..R7] that torch.manual_seed(seed); torch.randint(0, 45007, (7,)) yields
# (python/rz_linear/RzLinear.py:68-74), recorded here so that the oracle does not need torch.
HASH_CONSTANTS = {
    1024: [45007, 20011, 38363, 15263, 24507, 36489, 12234, 43027],
    0: [45007, 29440, 22221, 32190, 14791, 1316, 35275, 26448],
    1: [45007, 42280, 10019, 33951, 40424, 41193, 34731, 11534],
    42: [45007, 42355, 8976, 26801, 43886, 16055, 1500, 13717],
}


# ------------------------------------------------------------------ numpy restatement
LEGACY_PRIME = 2038074743
HASH_LEGACY = 3


def legacy_constants(seed):
    """[R0..R7] of the legacy generation for `seed` (/RzLinear.py:70-75): the prime, then odd
    numbers from numpy's RandomState(seed).randint(0, prime, 50) (an even draw is bumped by 1).
    Only R0..R3 enter its tile hash."""
    x = np.random.RandomState(seed).randint(0, LEGACY_PRIME, (50,))
    x = x + 1 * (x % 2 == 0)
    return [LEGACY_PRIME] + [int(v) for v in x[:7]]


def tile_offset(tk, tn, H, BK, BN, R, hash_levels=2):
    """Offset of tile (tk, tn) in hashed_weight, Python integers (no overflow possible).
    Two-level: RzLinearForward.py:316; one-level: RzLinearIdx.py:70-71; 3 = the legacy
    generation's tile hash, one level with range H - BK*BN + 1 (/rz_linear_kernel.cu:34-36,:56-64,
    where the tile is 16 x 16)."""
    R = [int(v) for v in R]
    if hash_levels == HASH_LEGACY:
        assert H >= BK * BN
        return ((tk * R[3] + tn * R[2] + R[1]) % R[0]) % (H - BK * BN + 1)
    rng = H - BK * BN
    assert rng > 0, "need H > BK*BN (RzLinearForward.py:28)"
    hi = (tk * R[3] + tn * R[2] + R[1]) % R[0]
    if hash_levels == 1:
        return hi % rng
    lo = (tk * R[7] + tn * R[5] + R[4]) % R[0]
    return (hi * R[0] + lo) % rng


def tile_offsets(K, N, H, BK, BN, R, hash_levels=2):
    TK, TN = -(-K // BK), -(-N // BN)
    out = np.empty((TK, TN), dtype=np.int64)
    for tk in range(TK):
        for tn in range(TN):
            out[tk, tn] = tile_offset(tk, tn, H, BK, BN, R, hash_levels)
    return out


def index_map(K, N, H, BK, BN, R, hash_levels=2):
    """int64 [K, N]: position in hashed_weight of W[k, n] (RzLinearForward.py:312-313)."""
    offs = tile_offsets(K, N, H, BK, BN, R, hash_levels)
    k = np.arange(K)[:, None]
    n = np.arange(N)[None, :]
    return offs[k // BK, n // BN] + (k % BK) * BN + (n % BN)


def materialize(hw, K, N, BK, BN, R, hash_levels=2):
    hw = np.asarray(hw, dtype=np.float64)
    return hw[index_map(K, N, hw.shape[0], BK, BN, R, hash_levels)]


def forward(X, hw, N, BK, BN, R, init_factor=1.0, hash_levels=2):
    X = np.asarray(X, dtype=np.float64)
    W = materialize(hw, X.shape[1], N, BK, BN, R, hash_levels)
    return (X @ W) * init_factor


def input_grad(dY, hw, K, BK, BN, R, init_factor=1.0, hash_levels=2):
    dY = np.asarray(dY, dtype=np.float64)
    W = materialize(hw, K, dY.shape[1], BK, BN, R, hash_levels)
    return (dY @ W.T) * init_factor


def weight_grad(X, dY, H, BK, BN, R, init_factor=1.0, hash_levels=2):
    X = np.asarray(X, dtype=np.float64)
    dY = np.asarray(dY, dtype=np.float64)
    K, N = X.shape[1], dY.shape[1]
    dW = X.T @ dY
    idx = index_map(K, N, H, BK, BN, R, hash_levels)
    return np.bincount(idx.ravel(), weights=dW.ravel(), minlength=H) * init_factor


# ------------------------------------------------------------------ C restatement
_lib = None


def build_c():
    """Compile oracle/rz_oracle.c with gcc (make)."""
    subprocess.run(["make", "-C", _DIR, "-s"], check=True)
    return _SO


def _c():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build_c()
        lib = ctypes.CDLL(_SO)
        i64, dp, i32p = ctypes.c_int64, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int32)
        lib.rz_oracle_tile_offset.restype = i64
        lib.rz_oracle_tile_offset.argtypes = [i64, i64, i64, i64, i64, i32p, ctypes.c_int]
        lib.rz_oracle_tile_offsets.restype = ctypes.c_int
        lib.rz_oracle_tile_offsets.argtypes = [ctypes.POINTER(i64), i64, i64, i64, i64, i64, i32p, ctypes.c_int]
        lib.rz_oracle_materialize.restype = ctypes.c_int
        lib.rz_oracle_materialize.argtypes = [dp, dp, i64, i64, i64, i64, i64, i32p, ctypes.c_int]
        for name in ("rz_oracle_forward", "rz_oracle_input_grad", "rz_oracle_weight_grad"):
            fn = getattr(lib, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [dp, dp, dp, i64, i64, i64, i64, i64, i64, i32p, ctypes.c_double]
        _lib = lib
    return _lib


def _r(R):
    return (ctypes.c_int32 * 8)(*[int(v) for v in R])


def _d(a):
    a = np.ascontiguousarray(a, dtype=np.float64)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def c_tile_offsets(K, N, H, BK, BN, R, hash_levels=2):
    TK, TN = -(-K // BK), -(-N // BN)
    out = np.empty((TK, TN), dtype=np.int64)
    st = _c().rz_oracle_tile_offsets(out.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), K, N, H, BK, BN,
                                     _r(R), hash_levels)
    if st != 0:
        raise ValueError("rz_oracle_tile_offsets status %d" % st)
    return out


def c_materialize(hw, K, N, BK, BN, R, hash_levels=2):
    hw, hp = _d(hw)
    W = np.empty((K, N), dtype=np.float64)
    st = _c().rz_oracle_materialize(hp, W.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), K, N, hw.shape[0],
                                    BK, BN, _r(R), hash_levels)
    assert st == 0, st
    return W


def c_forward(X, hw, N, BK, BN, R, init_factor=1.0):
    X, xp = _d(X)
    hw, hp = _d(hw)
    M, K = X.shape
    Y = np.empty((M, N), dtype=np.float64)
    st = _c().rz_oracle_forward(xp, hp, Y.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), M, K, N,
                                hw.shape[0], BK, BN, _r(R), float(init_factor))
    assert st == 0, st
    return Y


def c_input_grad(dY, hw, K, BK, BN, R, init_factor=1.0):
    dY, gp = _d(dY)
    hw, hp = _d(hw)
    M, N = dY.shape
    dX = np.empty((M, K), dtype=np.float64)
    st = _c().rz_oracle_input_grad(gp, hp, dX.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), M, K, N,
                                   hw.shape[0], BK, BN, _r(R), float(init_factor))
    assert st == 0, st
    return dX


def c_weight_grad(X, dY, H, BK, BN, R, init_factor=1.0):
    X, xp = _d(X)
    dY, gp = _d(dY)
    M, K = X.shape
    N = dY.shape[1]
    dHW = np.empty((H,), dtype=np.float64)
    st = _c().rz_oracle_weight_grad(xp, gp, dHW.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), M, K, N, H,
                                    BK, BN, _r(R), float(init_factor))
    assert st == 0, st
    return dHW
