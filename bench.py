#!/usr/bin/env python3
"""Benchmark of the RzLinear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--dtype bf16|fp32|fp16]

One step = one pass of the hot path over one batch that is already resident in HBM: forward
Y = X.W, input-grad dX = dY.W^T and weight-grad dHW = scatter_add(X^T.dY), each through the
C ABI of librzlinear.so with caller-owned, pre-allocated outputs.  The default workload is the
one the headline metric is quoted on: M = N = K = 4096, 1000x compression (H = 16778), bf16,
64x64 hashed tiles.  Prints ONE JSON line: fwd+bwd TFLOP/s (6*M*N*K flop per step), the
roofline of the slowest of the three kernels, the dense torch.matmul (hipBLASLt/rocBLAS) rate on
the same GPU under the same warm-up / step counts, a short sweep over the other baseline
configurations and the reference's CPU path timed on the host cores.

Order of the GPU work (the GPU's clock governor needs tens of milliseconds of load to settle after
an idle period, so what runs when is part of the protocol and is reported):
  output check -> clock settling (untimed, independent of --warmup: dense and rz legs alternate
  until three consecutive passes take the same time to within 2 %, at most 0.3 s) -> dense legs
  (W warm-up + K timed) -> rz legs (W warm-up + K timed: the headline) -> dense legs again (W + K)
  -> sweep (each row settles the same way first) -> practical MFMA ceiling -> CPU baseline.
The dense rate quoted against the headline is the mean of the two dense runs around it;
`rz_over_dense_settled` is against the faster of the two.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HASH_SEED_1024 = [45007, 20011, 38363, 15263, 24507, 36489, 12234, 43027]

# name -> (M, K, N, H, default dtype, input distributions[, (BLOCK_K, BLOCK_N)]); tiles are 64x64 (what the
# baseline configurations ask for) except on the reference's own grid, which runs its launchers' defaults.
# "normal": X ~ N(0,1), dY ~ N(0,1); "relu": X = relu(N(0,1)), dY ~ N(0, variance 1e-2).
WORKLOADS = {
    "square4096": (4096, 4096, 4096, 16778, "bf16", "normal"),      # the metric's configuration
    "square2048": (2048, 2048, 2048, 16384, "bf16", "normal"),
    "square1024": (1024, 1024, 1024, 16384, "bf16", "normal"),
    "cpu_ref_1024": (1024, 1024, 1024, 65536, "fp32", "normal"),
    "rec_mlp": (16384, 512, 1024, 5243, "bf16", "relu"),
    "ffn": (8192, 4096, 16384, 67109, "bf16", "normal"),
    "collision": (32768, 2048, 2048, 32768, "fp32", "normal"),
    # the shape grid of the reference's own benchmark script (python/bench/bench.py:10-11), with its
    # default compress_ratio 0.0625 and its launchers' default tile (BLOCK_SIZE_K = 32, BLOCK_SIZE_N = 64)
    "grid_32_1024": (32, 1024, 1024, 65536, "fp32", "normal", (32, 64)),
    "grid_128_1024": (128, 1024, 1024, 65536, "fp32", "normal", (32, 64)),
    "grid_1024_1024": (1024, 1024, 1024, 65536, "fp32", "normal", (32, 64)),
    "grid_32_10240": (32, 10240, 10240, 6553600, "fp32", "normal", (32, 64)),
    "grid_128_10240": (128, 10240, 10240, 6553600, "fp32", "normal", (32, 64)),
    "grid_1024_10240": (1024, 10240, 10240, 6553600, "fp32", "normal", (32, 64)),
}
# the baseline configurations beside the headline one: (workload, dtype) rows of the sweep
SWEEP = [("cpu_ref_1024", "fp32"), ("square1024", "fp32"), ("square1024", "bf16"), ("square2048", "fp32"),
         ("square2048", "bf16"), ("square4096", "fp32"), ("square4096", "bf16"), ("square4096", "fp16"),
         ("rec_mlp", "bf16"), ("ffn", "bf16"), ("collision", "fp32"),
         # the reference's own benchmark grid at its large size (python/bench/bench.py:10-11 runs it in fp32)
         ("grid_32_10240", "fp32"), ("grid_128_10240", "fp32"), ("grid_1024_10240", "fp32"),
         ("grid_32_10240", "bf16"), ("grid_128_10240", "bf16"), ("grid_1024_10240", "bf16")]
# dense MFMA peaks of MI355X, TFLOP/s
PEAK = {"bf16": 2500.0, "fp16": 2500.0, "fp32": 157.3}
# HBM bytes per launch of each leg, from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (KiB per
# dispatch, one run each), scaled by what the same counters read for a plain 256 MiB copy
# (FETCH_SIZE x2.0, WRITE_SIZE x1.0).  A counter run cannot be taken inside this script, so the
# figures are read off the committed summary named here; they describe the kernels of that
# summary and are dropped (null) for a workload that has none.
TRAFFIC = {
    # HBM bytes per launch of the contraction kernel of each leg: FETCH_SIZE * 2.0 + WRITE_SIZE * 1.0 KiB
    # (factors from the copy calibration at the end of every profile: a 256 MiB device copy reads back
    #  FETCH_SIZE = 131085, WRITE_SIZE = 262144)
    ("square4096", "bf16"): {
        "profile": "profiles/rz_gemm_bf16_square4096.txt",
        "bytes": {"forward": int((16679.6 * 2.0 + 32768.0) * 1024),       # algorithmic: 64.03 MiB
                  "input_grad": int((16676.4 * 2.0 + 32768.0) * 1024),
                  "weight_grad": int((98478.0 * 2.0 + 16784.6) * 1024)},  # X, dY re-read by the XCDs' tile groups; + partial images
    },
    ("square2048", "bf16"): {
        "profile": "profiles/rz_gemm_bf16_square2048.txt",
        "bytes": {"forward": int((4349.3 * 2.0 + 8192.0) * 1024), "input_grad": int((4342.2 * 2.0 + 8192.0) * 1024),
                  "weight_grad": int((24699.1 * 2.0 + 16384.0) * 1024)},
    },
    ("square4096", "fp32"): {
        "profile": "profiles/rz_gemm_fp32_square4096.txt",
        "bytes": {"forward": int((33229.8 * 2.0 + 65536.0) * 1024),       # algorithmic: 128.06 MiB
                  "input_grad": int((33225.7 * 2.0 + 65536.0) * 1024),
                  "weight_grad": int((196812.8 * 2.0 + 16784.7) * 1024)},
    },
    ("cpu_ref_1024", "fp32"): {
        "profile": "profiles/rz_gemm_fp32_cpu_ref_1024.txt",
        "bytes": {"forward": int((3160.8 * 2.0 + 4096.0) * 1024), "input_grad": int((3159.0 * 2.0 + 4096.0) * 1024),
                  "weight_grad": int((12338.6 * 2.0 + 4096.0) * 1024)},   # X^T.dY written tile by tile: 4 MiB
    },
    ("ffn", "bf16"): {
        "profile": "profiles/rz_gemm_fold_bf16_ffn.txt",
        "bytes": {"forward": int((70690.9 * 2.0 + 262144.0) * 1024),      # algorithmic: 320.1 MiB
                  "input_grad": int((132331.1 * 2.0 + 65536.0) * 1024),
                  # contraction (X, dY re-read by the XCDs' tile groups; X^T.dY written tile by tile in bf16: 128 MiB)
                  "weight_grad": int((786599.9 * 2.0 + 131072.0) * 1024)},
    },
    ("grid_1024_10240", "bf16"): {
        "profile": "profiles/rz_gemm_fold_bf16_grid_1024_10240.txt",
        "bytes": {"forward": int((396677.9 * 2.0 + 143380.0) * 1024),     # (three slices: fp32 partial planes written, read back by the slice that finishes)
                  "input_grad": int((382509.1 * 2.0 + 143380.1) * 1024),
                  "weight_grad": int((172198.8 * 2.0 + 204800.0) * 1024)},      # (X^T.dY tile by tile in bf16: 200 MiB)
    },
}


def make_workload(torch, _lib, name, dname, dev):
    """Resident inputs, outputs and workspaces of one workload and its three legs."""
    M, K, N, H, _, dist = WORKLOADS[name][:6]
    BK, BN = WORKLOADS[name][6] if len(WORKLOADS[name]) > 6 else (64, 64)
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[dname]
    code = {"bf16": _lib.RZ_BF16, "fp16": _lib.RZ_F16, "fp32": _lib.RZ_F32}[dname]
    lib = _lib.load()
    R = (ctypes.c_int32 * 8)(*HASH_SEED_1024)
    g = torch.Generator().manual_seed(1024)
    x = torch.randn((M, K), generator=g)
    hw = ((torch.rand((H,), generator=g) * 2 - 1) / K ** 0.5).to(dtype).to(dev)
    dy = torch.randn((M, N), generator=g)
    if dist == "relu":
        x, dy = torch.relu(x), dy * 0.1
    x, dy = x.to(dtype).to(dev), dy.to(dtype).to(dev)
    y = torch.empty((M, N), dtype=dtype, device=dev)
    dx = torch.empty((M, K), dtype=dtype, device=dev)
    dhw = torch.empty((H,), dtype=dtype, device=dev)
    ws_bytes = lib.rz_weight_grad_workspace_bytes(M, K, N, H, BK, BN, code)
    ws = torch.empty((max(ws_bytes, 16),), dtype=torch.uint8, device=dev)
    # skinny workloads split the contraction of forward / input-grad (0 bytes = no split)
    fws_bytes = lib.rz_forward_workspace_bytes(M, K, N, H, BK, BN, code)
    iws_bytes = lib.rz_input_grad_workspace_bytes(M, K, N, H, BK, BN, code)
    fws = torch.empty((max(fws_bytes, 16),), dtype=torch.uint8, device=dev)
    iws = torch.empty((max(iws_bytes, 16),), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def fwd():
        _lib.check(lib.rz_forward_ws(x.data_ptr(), hw.data_ptr(), None, y.data_ptr(), fws.data_ptr(), fws_bytes,
                                     M, K, N, H, BK, BN, R, 1.0, K, N, code, stream))

    def igrad():
        _lib.check(lib.rz_input_grad_ws(dy.data_ptr(), hw.data_ptr(), dx.data_ptr(), iws.data_ptr(), iws_bytes,
                                        M, K, N, H, BK, BN, R, 1.0, N, K, code, stream))

    # A hashed_weight too large for an LDS image: the layer's plan (tile offsets and window lists, a
    # function of the layer's constants alone, built once like the hash constants themselves and
    # kept on the device) goes with every call, as the package's own launchers do it.
    plan = None
    if _lib.plan_query(2, M, K, N, H, BK, BN, code, planned=True)["mode"] in ("window", "fold"):
        plan = _lib.layer_plan(K, N, H, BK, BN, R, 2, dev)

    def wgrad():
        if plan is not None:
            _lib.check(lib.rz_weight_grad_planned(x.data_ptr(), dy.data_ptr(), dhw.data_ptr(), None, ws.data_ptr(), ws_bytes,
                                                  plan.data_ptr(), plan.numel() * 4, M, K, N, H, BK, BN, R, 2, 1.0, K, N,
                                                  code, 0, None, stream))
        else:
            _lib.check(lib.rz_weight_grad(x.data_ptr(), dy.data_ptr(), dhw.data_ptr(), ws.data_ptr(), ws_bytes,
                                          M, K, N, H, BK, BN, R, 1.0, K, N, code, stream))

    # the dense products of the same shapes, each in the operand layout that is fastest for
    # the library (all "NN"), into pre-allocated outputs
    w = torch.randn((K, N), generator=g).to(dtype).to(dev)
    wt = w.t().contiguous()
    xt = x.t().contiguous()
    yd = torch.empty((M, N), dtype=dtype, device=dev)
    dxd = torch.empty((M, K), dtype=dtype, device=dev)
    dwd = torch.empty((K, N), dtype=dtype, device=dev)
    dense_legs = (("forward", lambda: torch.matmul(x, w, out=yd)),
                  ("input_grad", lambda: torch.matmul(dy, wt, out=dxd)),
                  ("weight_grad", lambda: torch.matmul(xt, dy, out=dwd)))
    wl = dict(M=M, K=K, N=N, H=H, BK=BK, BN=BN, R=R, code=code, dtype=dtype, dname=dname, x=x, hw=hw, dy=dy, y=y,
              dx=dx, dhw=dhw, layer_plan=plan is not None, legs=(("forward", fwd), ("input_grad", igrad), ("weight_grad", wgrad)),
              dense_legs=dense_legs, flop_gemm=2.0 * M * N * K)
    return wl


EVENT_EVERY = 4   # steps between two steps whose legs are bracketed by HIP events


def algorithmic_bytes(wl):
    """Least HBM bytes of each leg: forward s(MK + MN + H), input-grad s(MN + MK + H), weight-grad
    s(MK + MN) + 4H (the gradient is summed in fp32), s = bytes per element."""
    M, K, N, H = (wl[k] for k in ("M", "K", "N", "H"))
    s = 4 if wl["dname"] == "fp32" else 2
    return {"forward": s * (M * K + M * N + H), "input_grad": s * (M * N + M * K + H),
            "weight_grad": s * (M * K + M * N) + 4 * H}


def settle(torch, leg_sets, cap_s=0.3, agree=0.02):
    """Untimed: passes over every leg of `leg_sets` (dense and rz alternating, so that neither finds the
    clocks as the other left them) until three consecutive passes take the same time to within
    `agree`, for at most `cap_s` seconds.  Returns (passes, ms of the last pass)."""
    legs = [f for legs in leg_sets for _, f in legs]
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    last, t_end, n = [], time.perf_counter() + cap_s, 0
    while True:
        a.record()
        for f in legs:
            f()
        b.record()
        b.synchronize()
        n += 1
        last = (last + [a.elapsed_time(b)])[-3:]
        if (len(last) == 3 and max(last) <= min(last) * (1.0 + agree)) or time.perf_counter() >= t_end:
            return n, last[-1]


def run_legs(torch, legs, warmup, steps):
    """`warmup` untimed steps, then exactly `steps` timed ones between two synchronisations.  Every
    EVENT_EVERY-th timed step has HIP events on the launch stream around each of its legs (an event
    record is a packet of its own in the queue: around every leg of every step the records cost
    about 14 us per step of the metric configuration, 4 % — measurement, not hot path — so the
    other steps run without).  Returns (ms per step by the host clock, {leg: mean ms by the events})."""
    for _ in range(warmup):
        for _, f in legs:
            f()
    probed = [s for s in range(steps) if s % EVENT_EVERY == 0]
    ev = {s: [torch.cuda.Event(enable_timing=True) for _ in range(len(legs) + 1)] for s in probed}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        e = ev.get(s)
        if e is None:
            for _, f in legs:
                f()
        else:
            e[0].record()
            for i, (_, f) in enumerate(legs):
                f()
                e[i + 1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    leg_ms = {name: sum(ev[s][i].elapsed_time(ev[s][i + 1]) for s in probed) / len(probed)
              for i, (name, _) in enumerate(legs)}
    return (t1 - t0) * 1e3 / steps, leg_ms


def output_check(torch, _lib, wl):
    """One pass of the three legs checked on the GPU against W materialised by rz_materialize and
    torch's own products (float32 accumulate): a guard against timing a broken kernel, not the
    parity test (that is tests/, against the oracle).  Returns the normalised max errors."""
    lib = _lib.load()
    M, K, N, H, BK, BN = (wl[k] for k in ("M", "K", "N", "H", "BK", "BN"))
    stream = torch.cuda.current_stream().cuda_stream
    idx = torch.empty((K, N), dtype=torch.float32, device=wl["x"].device)
    ar = torch.arange(H, dtype=torch.float32, device=wl["x"].device)
    _lib.check(lib.rz_materialize(ar.data_ptr(), idx.data_ptr(), K, N, H, BK, BN, wl["R"], 2, N, _lib.RZ_F32, stream))
    idx = idx.long()
    for _, f in wl["legs"]:
        f()
    W = wl["hw"].float()[idx]
    xf, dyf = wl["x"].float(), wl["dy"].float()
    rel = lambda out, ref: float((out.float() - ref).abs().max() / ref.abs().max())
    errs = {"forward": rel(wl["y"], xf @ W), "input_grad": rel(wl["dx"], dyf @ W.t())}
    dW = xf.t() @ dyf
    ref = torch.zeros((H,), dtype=torch.float32, device=dW.device).index_add_(0, idx.reshape(-1), dW.reshape(-1))
    errs["weight_grad"] = rel(wl["dhw"], ref)
    torch.cuda.synchronize()
    tol = 1e-3 if wl["dname"] == "fp32" else 2e-2   # (the fp32 comparator is itself an fp32 product)
    bad = {k: v for k, v in errs.items() if not v <= tol}
    if bad:
        sys.exit("bench.py: output check failed, refusing to time: %s" % bad)
    return {k: float("%.3g" % v) for k, v in errs.items()}


def api_level(torch, wl, warmup, steps):
    """ms per forward + backward of rzlinear_amd.RzLinear (bias fused into the forward store, bias
    gradient from the weight-grad pass, gradients allocated by autograd) and of torch.nn.Linear,
    `warmup` + `steps` calls each, HIP events around the whole run."""
    from rzlinear_amd import RzLinear
    M, K, N, H, BK, BN = (wl[k] for k in ("M", "K", "N", "H", "BK", "BN"))
    dev, dtype = wl["x"].device, wl["dtype"]
    layer = RzLinear(K, N, hashed_weight=torch.nn.Parameter(wl["hw"].clone()), seed=1024, bias=True, dtype=dtype,
                     block_size_k=BK, block_size_n=BN).to(dev)
    dense = torch.nn.Linear(K, N, bias=True, dtype=dtype, device=dev)
    x = wl["x"].clone().requires_grad_(True)
    dy = wl["dy"]

    def run(mod):
        def step():
            x.grad = None
            for prm in mod.parameters():
                prm.grad = None
            mod(x).backward(dy)
        for _ in range(warmup):
            step()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(steps):
            step()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / steps

    d_ms = run(dense)
    rz_ms = run(layer)
    fl = 3 * wl["flop_gemm"]
    return {"what": "RzLinear module forward + backward through autograd (bias, bias gradient, allocations included), "
                    "%d + %d steps; torch.nn.Linear the same way" % (warmup, steps),
            "rz_ms": round(rz_ms, 4), "rz_tflops": round(tflops(fl, rz_ms), 2),
            "nn_linear_ms": round(d_ms, 4), "nn_linear_tflops": round(tflops(fl, d_ms), 2),
            "rz_over_nn_linear": round(d_ms / rz_ms, 4)}


def mfma_ceiling(torch, _lib, wl, launches=100):
    """The MFMA rate this GPU sustains on the matrix work alone of one contraction of the headline
    shape, with operands distributed like the workload's: rz_mfma_probe runs the inner loop's
    MFMA stream (256 workgroups of eight wavefronts, 32 MFMA 32x32x16 per wavefront and step, as
    many steps as make 2*M*N*K flop) without global loads, hashing or stores — mode 0 out of
    registers, mode 1 with the fragment reads from LDS and the barrier per step.  The gap between
    these figures and the data sheet's peak is the clock under matrix load (reported), not the
    kernels'.  16-bit types only."""
    if wl["dname"] == "fp32":
        return None
    lib = _lib.load()
    dev = wl["x"].device
    stream = torch.cuda.current_stream(dev).cuda_stream
    operands = wl["x"].reshape(-1)[:32768].contiguous()           # 64 KB of the workload's own X
    wgs = 256
    steps = max(1, int(round(wl["flop_gemm"] / (wgs * 8 * 32 * 32768.0))))
    out = torch.empty((wgs * 512,), dtype=torch.float32, device=dev)
    ticks = torch.zeros((2 * wgs,), dtype=torch.int64, device=dev)
    res = {"what": "rz_mfma_probe: %d workgroups x 8 wavefronts x %d steps x 32 MFMA 32x32x16 (%.1f GFLOP per launch), operands = "
                   "the workload's X; %d launches after as many untimed" % (wgs, steps, wgs * 8 * steps * 32 * 32768 / 1e9, launches)}
    for mode, key in ((0, "registers_only"), (1, "with_lds_fragments_and_barrier")):
        def launch():
            _lib.check(lib.rz_mfma_probe(operands.data_ptr(), out.data_ptr(), ticks.data_ptr(), wgs, steps, mode, wl["code"], stream))
        for _ in range(launches):
            launch()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(launches):
            launch()
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / launches
        t = ticks.view(wgs, 2).double().mean(0)
        res[key] = {"us_per_launch": round(ms * 1e3, 2), "tflops": round(tflops(wgs * 8 * steps * 32 * 32768.0, ms), 1),
                    "shader_clock_mhz": round(float(t[0] / (t[1] / 100.0)), 0)}
    return res


def tflops(flop, ms):
    return flop / (ms * 1e-3) / 1e12


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="square4096", choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default=None, choices=["bf16", "fp16", "fp32"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dense", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--no-api", action="store_true", help="skip the module-level (autograd) timing")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the MFMA-only probe (practical ceiling)")
    ap.add_argument("--cpu-budget", type=float, default=15.0, help="seconds of CPU-path timing")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="only run a plain device-to-device copy of this many MiB (five launches) and exit: "
                         "the known traffic against which rocprofv3's FETCH_SIZE / WRITE_SIZE are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (no collectives, no sharding); run with --gpus 1")

    import torch
    from rzlinear_amd import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    _lib.load()   # raises if librzlinear.so is not built: there is no fallback
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_copy > 0:
        n = args.calibrate_copy * 1024 * 1024
        src = torch.empty((n,), dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes_read": n, "calibrate_copy_bytes_written": n, "launches": 5}))
        return

    dname = args.dtype or WORKLOADS[args.workload][4]
    wl = make_workload(torch, _lib, args.workload, dname, dev)
    M, K, N, H, BK, BN = (wl[k] for k in ("M", "K", "N", "H", "BK", "BN"))
    flop_gemm = wl["flop_gemm"]
    peak = PEAK[dname]

    check = None if args.no_check else output_check(torch, _lib, wl)

    settled = settle(torch, [wl["legs"]] if args.no_dense else [wl["dense_legs"], wl["legs"]])

    dense_runs = []
    if not args.no_dense:
        dense_runs.append(run_legs(torch, wl["dense_legs"], args.warmup, args.steps))

    # ---- the headline: W warm-up steps, then exactly K timed steps ----------------------------
    ms_per_step, leg_ms = run_legs(torch, wl["legs"], args.warmup, args.steps)
    value = tflops(3 * flop_gemm, ms_per_step)

    if not args.no_dense:
        dense_runs.append(run_legs(torch, wl["dense_legs"], args.warmup, args.steps))

    leg_tflops = {k: tflops(flop_gemm, v) for k, v in leg_ms.items()}
    slowest = max(leg_ms, key=leg_ms.get)
    traffic = TRAFFIC.get((args.workload, dname))
    roofline = {
        "kernel": "rz_gemm_kernel<%s> (%s)" % (dname, slowest),
        "bound": "mfma",
        "achieved": round(leg_tflops[slowest], 2),
        "peak": peak,
        "unit": "TFLOP/s",
        "frac": round(leg_tflops[slowest] / peak, 4),
        "traffic": traffic["bytes"][slowest] if traffic else None,
        "traffic_source": traffic["profile"] if traffic else None,
        "per_kernel_tflops": {k: round(v, 2) for k, v in leg_tflops.items()},
        "per_kernel_ms": {k: round(v, 4) for k, v in leg_ms.items()},
    }

    dense = None
    if dense_runs:
        d_ms = {k: sum(r[1][k] for r in dense_runs) / len(dense_runs) for k in leg_ms}
        d_step = sum(r[0] for r in dense_runs) / len(dense_runs)
        dense_step_tf = tflops(3 * flop_gemm, d_step)
        dense = {
            "library": "torch.matmul (hipBLASLt/rocBLAS), operands pre-laid-out NN",
            "protocol": "same --warmup/--steps as the rz legs, once before and once after them; mean of the two",
            "per_kernel_tflops": {k: round(tflops(flop_gemm, v), 2) for k, v in d_ms.items()},
            "fwd_bwd_tflops": round(dense_step_tf, 2),
            "fwd_bwd_tflops_before_after": [round(tflops(3 * flop_gemm, r[0]), 2) for r in dense_runs],
            "rz_over_dense": round(value / dense_step_tf, 4),
            "rz_over_dense_settled": round(value / max(tflops(3 * flop_gemm, r[0]) for r in dense_runs), 4),
            "rz_over_dense_per_kernel": {k: round(d_ms[k] / leg_ms[k], 4) for k in leg_ms},
        }

    # ---- the other baseline configurations, short runs outside the headline's timed region ----
    sweep = None
    if not args.no_sweep:
        sweep = []
        sw_warm, sw_steps = 5, 20
        legs_of = ("forward", "input_grad", "weight_grad")
        for name, dn in SWEEP:
            if (name, dn) == (args.workload, dname):
                row_rz, row_d = (ms_per_step, leg_ms), None
                if dense_runs:
                    row_d = (d_step, d_ms)
                w2 = wl
            else:
                w2 = make_workload(torch, _lib, name, dn, dev)
                settle(torch, [w2["legs"]] if args.no_dense else [w2["dense_legs"], w2["legs"]], cap_s=0.15)
                row_d = run_legs(torch, w2["dense_legs"], sw_warm, sw_steps) if not args.no_dense else None
                row_rz = run_legs(torch, w2["legs"], sw_warm, sw_steps)
            fg = w2["flop_gemm"]
            row = {"workload": name, "dtype": dn, "M": w2["M"], "K": w2["K"], "N": w2["N"], "H": w2["H"],
                   "rz_tflops": {k: round(tflops(fg, v), 2) for k, v in row_rz[1].items()},
                   "rz_fwd_bwd_tflops": round(tflops(3 * fg, row_rz[0]), 2),
                   "pct_mfma_peak": round(100.0 * tflops(3 * fg, row_rz[0]) / PEAK[dn], 2),
                   # roofline fraction of the row's slowest leg (weight_grad = every kernel of the call)
                   "frac": round(min(tflops(fg, row_rz[1][k]) for k in legs_of) / PEAK[dn], 4),
                   "slowest": max(legs_of, key=lambda k: row_rz[1][k])}
            tr = TRAFFIC.get((name, dn))
            if tr:   # measured HBM bytes of the contraction kernel of each leg over the least possible
                alg = algorithmic_bytes(w2)
                row["traffic_over_algorithmic"] = {k: round(tr["bytes"][k] / alg[k], 2) for k in legs_of}
                row["traffic_source"] = tr["profile"]
            if row_d is not None:
                row["dense_tflops"] = {k: round(tflops(fg, v), 2) for k, v in row_d[1].items()}
                row["rz_over_dense"] = {k: round(row_d[1][k] / row_rz[1][k], 3) for k in row_rz[1]}
                row["rz_over_dense"]["fwd_bwd"] = round(row_d[0] / row_rz[0], 3)
            sweep.append(row)
            if w2 is not wl:
                del w2
                torch.cuda.empty_cache()
        sweep = {"protocol": "per configuration: clocks settled as for the headline (at most 0.15 s), then warm-up %d + %d "
                             "timed steps (dense legs first, then rz); the headline configuration's row repeats the "
                             "headline run; frac = slowest leg / MFMA peak of the dtype" % (sw_warm, sw_steps),
                 "rows": sweep}

    # ---- the same step through the package's module and autograd (what a user of the reference
    # calls: python/bench/bench.py:44 times `rz(a)`), outputs allocated by the API, beside
    # torch.nn.Linear of the same shape timed the same way; short, outside the headline ----------
    api = None
    if not args.no_api:
        api = api_level(torch, wl, 5, 20)

    ceiling = None if args.no_ceiling else mfma_ceiling(torch, _lib, wl)
    if ceiling is not None:
        roofline["practical_ceiling"] = ceiling
        roofline["frac_of_practical_ceiling"] = round(leg_tflops[slowest] / ceiling["registers_only"]["tflops"], 4)

    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import cpu_path   # checker/baseline only: never on the measured GPU path
        # every host core this job may use: the machine's, unless the job was given a smaller
        # share through OMP_NUM_THREADS (GPU boxes hand one GPU's job a share of the host)
        share = os.environ.get("OMP_NUM_THREADS")
        cores = os.cpu_count() or 1
        if share and share.isdigit() and int(share) > 0:
            cores = min(cores, int(share))
        torch.set_num_threads(cores)
        sec, reps = cpu_path.time_cpu_path(M, K, N, H, BK, BN, HASH_SEED_1024, budget_s=args.cpu_budget)
        cpu_baseline = {
            "value": round(3 * flop_gemm / sec / 1e12, 4),
            "unit": "TFLOP/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "same shape M=%d K=%d N=%d H=%d in fp32: hash-gather W + torch.matmul fwd+bwd, median of %d "
                      "steps (%.2f s each) on %d threads (host has %d cores, OMP_NUM_THREADS=%s)"
                      % (M, K, N, H, reps, sec, torch.get_num_threads(), os.cpu_count() or 1, share),
        }

    out = {
        "metric": "fwd+bwd TFLOP/s at M=%d K=%d N=%d, %.0fx compression; %% MFMA peak" % (M, K, N, K * N / H)
                  if args.workload != "square4096" else "fwd+bwd TFLOP/s at M=N=K=4096, 1000x compression; % MFMA peak",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dname,
        "data": "synthetic",
        "config": {"workload": "%s: M=%d K=%d N=%d H=%d BLOCK_K=%d BLOCK_N=%d %s, fwd + input-grad + weight-grad"
                               % (args.workload, M, K, N, H, BK, BN, dname),
                   "hash_seed": 1024, "init_factor": 1.0,
                   "weight_grad_layer_plan": bool(wl["layer_plan"])},
        "pct_mfma_peak": round(100.0 * value / peak, 2),
        "output_check": check,
        "clock_settling": {"passes": settled[0], "last_pass_ms": round(settled[1], 4),
                           "rule": "untimed passes over dense + rz legs until three in a row agree within 2 %, at most 0.3 s"},
        "roofline": roofline,
        "dense_gemm": dense,
        "api_level": api,
        "cpu_baseline": cpu_baseline,
        "sweep": sweep,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
