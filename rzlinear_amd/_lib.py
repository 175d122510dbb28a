"""ctypes binding of librzlinear.so (the gfx950 HIP kernels behind a C ABI).

The library is built in-tree by ``python -m rzlinear_amd.build``.  There is no CPU or
PyTorch fallback: if the shared object is missing, or a tensor is not on a ROCm device,
the operators raise.
"""
import ctypes
import os

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "librzlinear.so")

RZ_F32, RZ_BF16, RZ_F16 = 0, 1, 2
_DTYPES = {torch.float32: RZ_F32, torch.bfloat16: RZ_BF16, torch.float16: RZ_F16}

# every symbol that include/rzlinear.h declares
EXPORTS = (
    "rz_version", "rz_status_string", "rz_tile_offsets", "rz_tile_offsets_device", "rz_forward",
    "rz_forward_bias", "rz_forward_workspace_bytes", "rz_forward_ws", "rz_input_grad",
    "rz_input_grad_workspace_bytes", "rz_input_grad_ws", "rz_weight_grad_workspace_bytes", "rz_weight_grad", "rz_weight_grad_ex_workspace_bytes",
    "rz_weight_grad_ex", "rz_forward_hashed", "rz_input_grad_hashed", "rz_weight_grad_hashed", "rz_materialize",
    "rz_forward_hashed_workspace_bytes", "rz_input_grad_hashed_workspace_bytes",
    "rz_weight_grad_hashed_workspace_bytes", "rz_plan_query", "rz_weight_grad_static",
    "rz_layer_plan_bytes", "rz_layer_plan_build", "rz_weight_grad_planned",
    "rz_sgd_step", "rz_adam_step", "rz_mfma_probe",
)


class Tuning(ctypes.Structure):
    """struct rz_tuning of include/rzlinear.h: overrides of the library's own choices (all zero =
    automatic).  Only tests and benchmarks set any of it."""
    _fields_ = [("tile", ctypes.c_int), ("stages", ctypes.c_int), ("lds_image", ctypes.c_int),
                ("window", ctypes.c_int), ("split", ctypes.c_int), ("clamp", ctypes.c_int),
                ("fold", ctypes.c_int), ("fold_tiles", ctypes.c_int), ("finish", ctypes.c_int), ("poll_limit", ctypes.c_int)]


# What the launchers of this package pass as `tuning` (None = automatic).  The C library keeps no
# settings of its own; this module-level value is the Python side's, set with `tuning(...)`.
_tuning = None


class tuning:
    """Context manager: ``with _lib.tuning(tile=128, lds_image=-1): ...`` makes the launchers
    called inside pass these overrides to the library (see struct rz_tuning)."""

    def __init__(self, **fields):
        self._new = Tuning(**fields) if fields else None

    def __enter__(self):
        global _tuning
        self._old, _tuning = _tuning, self._new
        return self._new

    def __exit__(self, *exc):
        global _tuning
        _tuning = self._old
        return False


def current_tuning():
    """ctypes argument for the `tuning` parameter of the *_hashed entry points."""
    return ctypes.byref(_tuning) if _tuning is not None else None

_lib = None
_host_answers = {}


def host_query(name, *args):
    """lib.<name>(*args, tuning) for the host-only queries (workspace sizes), remembered per
    argument tuple and tuning: a layer asks the same question on every step, and the answer is a
    pure function of the arguments."""
    t = _tuning
    key = (name, args, None if t is None else tuple(getattr(t, f) for f, _ in Tuning._fields_))
    try:
        return _host_answers[key]
    except KeyError:
        if len(_host_answers) > 4096:
            _host_answers.clear()
        v = _host_answers[key] = getattr(load(), name)(*args, current_tuning())
        return v


class RzLinearError(RuntimeError):
    """A librzlinear entry point returned a non-zero status."""

    def __init__(self, status, message):
        super().__init__("librzlinear: %s (status %d)" % (message, status))
        self.status = status


def load():
    """Load librzlinear.so once and declare the argument types of its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "librzlinear.so is not built (%s missing); run `python -m rzlinear_amd.build`. "
            "rzlinear_amd has no fallback path." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    c_int, c_i64, c_f, c_vp, c_sz = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
    i32p = ctypes.POINTER(ctypes.c_int32)
    lib.rz_version.restype = c_int
    lib.rz_version.argtypes = []
    lib.rz_status_string.restype = ctypes.c_char_p
    lib.rz_status_string.argtypes = [c_int]
    lib.rz_tile_offsets.restype = c_int
    lib.rz_tile_offsets.argtypes = [i32p, c_int, c_int, c_int, c_int, c_int, i32p, c_int]
    lib.rz_tile_offsets_device.restype = c_int
    lib.rz_tile_offsets_device.argtypes = [c_vp, c_int, c_int, c_int, c_int, c_int, i32p, c_int, c_vp]
    lib.rz_forward.restype = c_int
    lib.rz_forward.argtypes = [c_vp, c_vp, c_vp, c_int, c_int, c_int, c_int, c_int, c_int, i32p, c_f,
                               c_i64, c_i64, c_int, c_vp]
    lib.rz_forward_bias.restype = c_int
    lib.rz_forward_bias.argtypes = [c_vp, c_vp, c_vp, c_vp, c_int, c_int, c_int, c_int, c_int, c_int, i32p,
                                    c_f, c_i64, c_i64, c_int, c_vp]
    lib.rz_input_grad.restype = c_int
    lib.rz_input_grad.argtypes = lib.rz_forward.argtypes
    lib.rz_forward_workspace_bytes.restype = c_sz
    lib.rz_forward_workspace_bytes.argtypes = [c_int] * 7
    lib.rz_input_grad_workspace_bytes.restype = c_sz
    lib.rz_input_grad_workspace_bytes.argtypes = [c_int] * 7
    lib.rz_forward_ws.restype = c_int
    lib.rz_forward_ws.argtypes = [c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_int, c_int, c_int, c_int, c_int, c_int,
                                  i32p, c_f, c_i64, c_i64, c_int, c_vp]
    lib.rz_input_grad_ws.restype = c_int
    lib.rz_input_grad_ws.argtypes = [c_vp, c_vp, c_vp, c_vp, c_sz, c_int, c_int, c_int, c_int, c_int, c_int,
                                     i32p, c_f, c_i64, c_i64, c_int, c_vp]
    lib.rz_weight_grad_workspace_bytes.restype = c_sz
    lib.rz_weight_grad_workspace_bytes.argtypes = [c_int] * 7
    lib.rz_weight_grad.restype = c_int
    lib.rz_weight_grad.argtypes = [c_vp, c_vp, c_vp, c_vp, c_sz, c_int, c_int, c_int, c_int, c_int, c_int,
                                   i32p, c_f, c_i64, c_i64, c_int, c_vp]
    lib.rz_weight_grad_static.restype = c_int
    lib.rz_weight_grad_static.argtypes = [c_vp, c_vp, c_vp, c_int, c_int, c_int, c_int, c_int, c_int,
                                          i32p, c_f, c_i64, c_i64, c_int, c_vp]
    lib.rz_weight_grad_ex_workspace_bytes.restype = c_sz
    lib.rz_weight_grad_ex_workspace_bytes.argtypes = [c_int] * 7 + [ctypes.c_uint, c_int]
    lib.rz_weight_grad_ex.restype = c_int
    lib.rz_weight_grad_ex.argtypes = [c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_int, c_int, c_int, c_int, c_int, c_int,
                                      i32p, c_f, c_i64, c_i64, c_int, ctypes.c_uint, c_vp]
    tun = ctypes.POINTER(Tuning)
    lib.rz_forward_hashed.restype = c_int
    lib.rz_forward_hashed.argtypes = [c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_int, c_int, c_int, c_int, c_int, c_int,
                                      i32p, c_int, c_f, c_i64, c_i64, c_int, tun, c_vp]
    lib.rz_input_grad_hashed.restype = c_int
    lib.rz_input_grad_hashed.argtypes = [c_vp, c_vp, c_vp, c_vp, c_sz, c_int, c_int, c_int, c_int, c_int, c_int,
                                         i32p, c_int, c_f, c_i64, c_i64, c_int, tun, c_vp]
    lib.rz_weight_grad_hashed.restype = c_int
    lib.rz_weight_grad_hashed.argtypes = [c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_int, c_int, c_int, c_int, c_int,
                                          c_int, i32p, c_int, c_f, c_i64, c_i64, c_int, ctypes.c_uint, tun, c_vp]
    lib.rz_forward_hashed_workspace_bytes.restype = c_sz
    lib.rz_forward_hashed_workspace_bytes.argtypes = [c_int] * 7 + [tun]
    lib.rz_input_grad_hashed_workspace_bytes.restype = c_sz
    lib.rz_input_grad_hashed_workspace_bytes.argtypes = [c_int] * 7 + [tun]
    lib.rz_weight_grad_hashed_workspace_bytes.restype = c_sz
    lib.rz_weight_grad_hashed_workspace_bytes.argtypes = [c_int] * 7 + [ctypes.c_uint, c_int, tun]
    lib.rz_layer_plan_bytes.restype = c_sz
    lib.rz_layer_plan_bytes.argtypes = [c_int] * 5
    lib.rz_layer_plan_build.restype = c_int
    lib.rz_layer_plan_build.argtypes = [c_vp, c_sz, c_int, c_int, c_int, c_int, c_int, i32p, c_int]
    lib.rz_weight_grad_planned.restype = c_int
    lib.rz_weight_grad_planned.argtypes = [c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_vp, c_sz, c_int, c_int, c_int,
                                           c_int, c_int, c_int, i32p, c_int, c_f, c_i64, c_i64, c_int,
                                           ctypes.c_uint, tun, c_vp]
    lib.rz_plan_query.restype = c_int
    lib.rz_plan_query.argtypes = [c_int] * 8 + [ctypes.c_uint, c_int, tun, i32p]
    f32p = c_vp
    lib.rz_sgd_step.restype = c_int
    lib.rz_sgd_step.argtypes = [c_vp, c_vp, f32p, f32p, c_i64, c_int, c_int, c_f, c_f, c_f, c_f, c_int, c_int, c_f, c_vp]
    lib.rz_adam_step.restype = c_int
    lib.rz_adam_step.argtypes = [c_vp, c_vp, f32p, f32p, f32p, c_i64, c_int, c_int, c_f, c_f, c_f, c_f, c_f, c_int,
                                 c_int, c_f, c_vp]
    lib.rz_mfma_probe.restype = c_int
    lib.rz_mfma_probe.argtypes = [c_vp, c_vp, c_vp, c_int, c_int, c_int, c_int, c_vp]
    lib.rz_materialize.restype = c_int
    lib.rz_materialize.argtypes = [c_vp, c_vp, c_int, c_int, c_int, c_int, c_int, i32p, c_int, c_i64,
                                   c_int, c_vp]
    _lib = lib
    return lib


# options of rz_weight_grad_ex
WG_ACCUMULATE, WG_DHW_F32, WG_DBIAS_F32 = 1, 2, 4
# tile hashes (rz_hash)
HASH_ONE_LEVEL, HASH_TWO_LEVEL, HASH_LEGACY = 1, 2, 3


def check(status):
    if status != 0:
        raise RzLinearError(status, load().rz_status_string(status).decode())


def hash_constants(R7, R6, R5, R4, R3, R2, R1, R0):
    """The eight hash constants as the int32[8] array the C ABI takes (index = subscript)."""
    return (ctypes.c_int32 * 8)(int(R0), int(R1), int(R2), int(R3), int(R4), int(R5), int(R6), int(R7))


def dtype_code(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError("rzlinear_amd supports float32, bfloat16 and float16, got %s" % t.dtype)


try:   # the raw handle of the current stream, without building a torch.cuda.Stream object around it
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:   # pragma: no cover
    def _raw_stream(index):
        return torch.cuda.current_stream(index).cuda_stream


def require_gpu(*tensors):
    """All tensors must live on one ROCm device; returns the raw HIP stream handle to use."""
    first = tensors[0]
    if not first.is_cuda:
        raise RuntimeError("rzlinear_amd runs on a ROCm GPU only; got a tensor on %s" % first.device)
    index = first.get_device()
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("rzlinear_amd runs on a ROCm GPU only; got a tensor on %s" % t.device)
        if t.get_device() != index:
            raise RuntimeError("rzlinear_amd: tensors on different devices (%s, %s)" % (first.device, t.device))
    return _raw_stream(index)


def rows(t):
    """A 2-D tensor with unit column stride (copied only if it has to be) and its row pitch."""
    if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    ld = t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)
    return t, ld


def workspace(nbytes, device):
    """A scratch buffer of nbytes on `device` (None when nbytes is 0)."""
    return torch.empty((nbytes,), device=device, dtype=torch.uint8) if nbytes else None


def tile_offsets(K, N, H, BLOCK_SIZE_K, BLOCK_SIZE_N, random_numbers, hash_levels=2):
    """Host-side tile offsets as an int32 tensor [ceil(K/BK), ceil(N/BN)] (bit-exact hash)."""
    lib = load()
    TK, TN = -(-K // BLOCK_SIZE_K), -(-N // BLOCK_SIZE_N)
    out = torch.empty((TK, TN), dtype=torch.int32)
    R = (ctypes.c_int32 * 8)(*[int(v) for v in random_numbers])
    check(lib.rz_tile_offsets(ctypes.cast(out.data_ptr(), ctypes.POINTER(ctypes.c_int32)), K, N, H,
                              BLOCK_SIZE_K, BLOCK_SIZE_N, R, hash_levels))
    return out


_layer_plans = {}
# Whether the weight-grad launchers take a layer plan where one helps (tests switch it off to reach
# the kernels' own search for their strips).
use_layer_plans = True


def clear_layer_plans():
    """Forget every layer plan built so far (they are kept per layer geometry and device until this
    is called; a process that goes through many geometries can release them here)."""
    _layer_plans.clear()


def layer_plan(K, N, H, BK, BN, R, hash_levels, device):
    """The layer plan (rz_layer_plan_build) for these layer constants as an int32 tensor on `device`,
    built on the host the first time it is asked for and kept until clear_layer_plans() (it depends
    on the layer alone: shapes, tile and hash constants; about 10 bytes per W tile strip).  The
    first request copies the plan to the device with an ordinary, synchronous copy: make it outside
    a stream capture (one warm-up call of the layer, or this function itself, does)."""
    key = (K, N, H, BK, BN, tuple(int(v) for v in R), int(hash_levels), str(device))
    plan = _layer_plans.get(key)
    if plan is None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("rzlinear_amd: the layer plan for K=%d N=%d H=%d tile %dx%d has to be built (a host-to-device "
                               "copy) but the current stream is being captured; call the layer once, or "
                               "_lib.layer_plan(...), before the capture" % (K, N, H, BK, BN))
        lib = load()
        nbytes = lib.rz_layer_plan_bytes(K, N, H, BK, BN)
        if nbytes == 0:
            raise ValueError("no layer plan for K=%d N=%d H=%d tile %dx%d" % (K, N, H, BK, BN))
        host = torch.empty((nbytes // 4,), dtype=torch.int32)
        check(lib.rz_layer_plan_build(host.data_ptr(), nbytes, K, N, H, BK, BN, R, hash_levels))
        plan = _layer_plans[key] = host.to(device)
    return plan


PLAN_MODES = {0: "store", 1: "split", 2: "lds_image", 3: "atomics", 4: "window", 5: "fold"}


PLAN_WITH_LAYER_PLAN = 0x100


def plan_query(op, M, K, N, H, BK, BN, dtype_code_, flags=0, with_dbias=False, planned=False):
    """How the library would carry out a call (rz_plan_query), under the current tuning:
    dict(tile, slices, slice_len, step, mode, workgroups, shares, windows).  op: 0 forward, 1 input-grad,
    2 weight-grad; planned: the call will carry a layer plan (rz_weight_grad_planned).  For mode "split",
    shares = 1 says that the kernel finishes its own tiles (no second kernel)."""
    t = _tuning
    if planned:
        flags |= PLAN_WITH_LAYER_PLAN
    key = ("rz_plan_query", (op, M, K, N, H, BK, BN, dtype_code_, flags, int(with_dbias)),
           None if t is None else tuple(getattr(t, f) for f, _ in Tuning._fields_))
    ans = _host_answers.get(key)
    if ans is None:
        out = (ctypes.c_int32 * 8)()
        check(load().rz_plan_query(op, M, K, N, H, BK, BN, dtype_code_, flags, int(with_dbias), current_tuning(), out))
        ans = _host_answers[key] = dict(tile=out[0], slices=out[1], slice_len=out[2], step=out[3],
                                        mode=PLAN_MODES[out[4]], workgroups=out[5], shares=out[6], windows=out[7])
    return dict(ans)
