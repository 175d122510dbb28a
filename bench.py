#!/usr/bin/env python3
"""Benchmark of the RzLinear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--dtype bf16|fp32|fp16]

One step = one pass of the hot path over one batch that is already resident in HBM: forward
Y = X.W, input-grad dX = dY.W^T and weight-grad dHW = scatter_add(X^T.dY), each through the
C ABI of librzlinear.so with caller-owned, pre-allocated outputs.  The default workload is the
one the headline metric is quoted on: M = N = K = 4096, 1000x compression (H = 16778), bf16,
64x64 hashed tiles.  Prints ONE JSON line: fwd+bwd TFLOP/s (6*M*N*K flop per step), the
roofline of the slowest of the three kernels, the dense torch.matmul (hipBLASLt/rocBLAS) rate on
the same GPU and the reference's CPU path timed on the host cores.
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

# name -> (M, K, N, H, default dtype); tiles are 64x64 throughout
WORKLOADS = {
    "square4096": (4096, 4096, 4096, 16778, "bf16"),      # the metric's configuration
    "square2048": (2048, 2048, 2048, 16384, "bf16"),
    "square1024": (1024, 1024, 1024, 16384, "bf16"),
    "cpu_ref_1024": (1024, 1024, 1024, 65536, "fp32"),
    "rec_mlp": (16384, 512, 1024, 5243, "bf16"),
    "ffn": (8192, 4096, 16384, 67109, "bf16"),
    "collision": (32768, 2048, 2048, 32768, "fp32"),
    # the shape grid of the reference's own benchmark script (python/bench/bench.py:10-11),
    # with its default compress_ratio 0.0625
    "grid_32_1024": (32, 1024, 1024, 65536, "fp32"),
    "grid_128_1024": (128, 1024, 1024, 65536, "fp32"),
    "grid_1024_1024": (1024, 1024, 1024, 65536, "fp32"),
    "grid_32_10240": (32, 10240, 10240, 6553600, "fp32"),
    "grid_128_10240": (128, 10240, 10240, 6553600, "fp32"),
    "grid_1024_10240": (1024, 10240, 10240, 6553600, "fp32"),
}
# dense MFMA peaks of MI355X, TFLOP/s
PEAK = {"bf16": 2500.0, "fp16": 2500.0, "fp32": 157.3}
# HBM bytes per launch, measured once with rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (KiB per
# dispatch) and scaled by what the same counters read for a plain 256 MiB copy (FETCH_SIZE x2.0,
# WRITE_SIZE x1.0); the rocprof summary with the raw readings is committed with the profiles.
TRAFFIC_BYTES = {
    ("square4096", "bf16"): {
        "forward": int((16672.7 * 2.0 + 32768.0) * 1024),       # algorithmic: 64.03 MiB
        "input_grad": int((16672.7 * 2.0 + 32768.0) * 1024),
        "weight_grad": int((98457.7 * 2.0 + 16785.8) * 1024),   # X, dY re-read by 3 XCD groups; + partial images
    },
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="square4096", choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default=None, choices=["bf16", "fp16", "fp32"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dense", action="store_true")
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
    lib = _lib.load()   # raises if librzlinear.so is not built: there is no fallback
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

    M, K, N, H, dflt = WORKLOADS[args.workload]
    dname = args.dtype or dflt
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[dname]
    code = {"bf16": _lib.RZ_BF16, "fp16": _lib.RZ_F16, "fp32": _lib.RZ_F32}[dname]
    BK = BN = 64
    R = (ctypes.c_int32 * 8)(*HASH_SEED_1024)

    g = torch.Generator().manual_seed(1024)
    x = torch.randn((M, K), generator=g).to(dtype).to(dev)
    hw = ((torch.rand((H,), generator=g) * 2 - 1) / K ** 0.5).to(dtype).to(dev)
    dy = torch.randn((M, N), generator=g).to(dtype).to(dev)
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

    def wgrad():
        _lib.check(lib.rz_weight_grad(x.data_ptr(), dy.data_ptr(), dhw.data_ptr(), ws.data_ptr(), ws_bytes,
                                      M, K, N, H, BK, BN, R, 1.0, K, N, code, stream))

    legs = (("forward", fwd), ("input_grad", igrad), ("weight_grad", wgrad))

    for _ in range(args.warmup):
        for _, f in legs:
            f()
    torch.cuda.synchronize()

    # timed region: exactly `steps` steps; HIP events on the launch stream around every leg
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(len(legs) + 1)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.steps):
        ev[s][0].record()
        for i, (_, f) in enumerate(legs):
            f()
            ev[s][i + 1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    flop_gemm = 2.0 * M * N * K
    value = 3 * flop_gemm / (ms_per_step * 1e-3) / 1e12

    leg_ms = {}
    for i, (name, _) in enumerate(legs):
        leg_ms[name] = sum(ev[s][i].elapsed_time(ev[s][i + 1]) for s in range(args.steps)) / args.steps
    leg_tflops = {k: flop_gemm / (v * 1e-3) / 1e12 for k, v in leg_ms.items()}
    slowest = max(leg_ms, key=leg_ms.get)
    peak = PEAK[dname]
    roofline = {
        "kernel": "rz_gemm_kernel<%s> (%s)" % (dname, slowest),
        "bound": "mfma",
        "achieved": round(leg_tflops[slowest], 2),
        "peak": peak,
        "unit": "TFLOP/s",
        "frac": round(leg_tflops[slowest] / peak, 4),
        "traffic": TRAFFIC_BYTES.get((args.workload, dname), {}).get(slowest),
        "per_kernel_tflops": {k: round(v, 2) for k, v in leg_tflops.items()},
        "per_kernel_ms": {k: round(v, 4) for k, v in leg_ms.items()},
    }

    dense = None
    if not args.no_dense:
        w = torch.randn((K, N), generator=g).to(dtype).to(dev)
        wt = w.t().contiguous()
        xt = x.t().contiguous()

        def timeit(fn, n=100):
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(n):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / n

        yd = torch.empty((M, N), dtype=dtype, device=dev)
        dxd = torch.empty((M, K), dtype=dtype, device=dev)
        dwd = torch.empty((K, N), dtype=dtype, device=dev)
        # each dense product in the operand layout that is fastest for the library (all "NN")
        d_ms = {
            "forward": timeit(lambda: torch.matmul(x, w, out=yd)),
            "input_grad": timeit(lambda: torch.matmul(dy, wt, out=dxd)),
            "weight_grad": timeit(lambda: torch.matmul(xt, dy, out=dwd)),
        }
        d_tf = {k: flop_gemm / (v * 1e-3) / 1e12 for k, v in d_ms.items()}
        dense_step = 3 * flop_gemm / (sum(d_ms.values()) * 1e-3) / 1e12
        dense = {
            "library": "torch.matmul (hipBLASLt/rocBLAS), operands pre-laid-out NN",
            "per_kernel_tflops": {k: round(v, 2) for k, v in d_tf.items()},
            "fwd_bwd_tflops": round(dense_step, 2),
            "rz_over_dense": round(value / dense_step, 4),
        }
        del w, wt, xt, yd, dxd, dwd

    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import cpu_path   # checker/baseline only: never on the measured GPU path
        torch.set_num_threads(min(os.cpu_count() or 1, 16))
        sec, reps = cpu_path.time_cpu_path(M, K, N, H, BK, BN, HASH_SEED_1024, budget_s=args.cpu_budget)
        cpu_baseline = {
            "value": round(3 * flop_gemm / sec / 1e12, 4),
            "unit": "TFLOP/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "same shape M=%d K=%d N=%d H=%d in fp32: hash-gather W + torch.matmul fwd+bwd, median of %d "
                      "steps (%.2f s each)" % (M, K, N, H, reps, sec),
        }

    out = {
        "metric": "fwd+bwd TFLOP/s at M=N=K=4096, 1000x compression; % MFMA peak",
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
                   "hash_seed": 1024, "init_factor": 1.0},
        "pct_mfma_peak": round(100.0 * value / peak, 2),
        "roofline": roofline,
        "dense_gemm": dense,
        "cpu_baseline": cpu_baseline,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
