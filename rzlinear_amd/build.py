"""Builds librzlinear.so (the gfx950 HIP kernels + C ABI) in-tree with hipcc.

    python -m rzlinear_amd.build          # compile every csrc/*.hip and link
    python -m rzlinear_amd.build --asm    # also keep the device assembly next to the objects

hipcc cross-compiles for gfx950 without a GPU present, so this runs on a CPU-only host.
"""
import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_PATH = os.path.join(PKG_DIR, "librzlinear.so")

ARCH = "gfx950"
# Packed-fp32 VALU forms are switched off for all device code of this library.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; librzlinear.so cannot be built")
    return exe


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src, keep_asm, extra=(), obj_dir=OBJ_DIR):
    obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
    cmd = [_hipcc()] + HIPCC_FLAGS + list(extra) + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    if keep_asm:
        asm = obj[:-2] + ".s"
        cmd = [_hipcc()] + HIPCC_FLAGS + list(extra) + ["--cuda-device-only", "-S", src, "-o", asm]
        subprocess.run(cmd, capture_output=True, text=True, check=True)
    return obj


def build(keep_asm=False, jobs=None, verbose=True, extra_flags=(), out=None):
    """Compile every HIP source and link librzlinear.so; returns its path.

    extra_flags / out build a variant (e.g. with -D tuning switches) next to the default one;
    set rzlinear_amd._lib.LIB_PATH to its path before the first call to load it."""
    out = out or LIB_PATH
    obj_dir = OBJ_DIR if out == LIB_PATH else os.path.join(OBJ_DIR, "variant_" + os.path.basename(out).replace(".", "_"))
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), os.cpu_count() or 1, 16)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, keep_asm, extra_flags, obj_dir), srcs))
    tmp = out + ".tmp"
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    os.replace(tmp, out)
    if verbose:
        print("built", out, "from", len(srcs), "sources")
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--asm", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    ap.add_argument("-o", "--out", default=None, help="build a variant library at this path")
    ap.add_argument("-D", action="append", default=[], help="extra preprocessor define (variant builds)")
    a = ap.parse_args()
    build(keep_asm=a.asm, jobs=a.j, extra_flags=["-D" + d for d in a.D], out=a.out)
    sys.exit(0)
