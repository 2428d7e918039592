"""Offline build of the native-hip library with hipcc for gfx950.

    python -m oxibonsai_amd.build

produces ``oxibonsai_amd/lib/liboxb_hip.so`` (loaded through ctypes / dlopen)
and ``oxibonsai_amd/lib/liboxb_hip.a`` (what a Rust build script links).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "lib")
SOURCES = ["runtime.hip", "gemv_kernels.hip", "gemm_kernels.hip", "layer_kernels.hip", "prefill_kernels.hip", "token_kernels.hip", "model.hip", "repack.cpp", "gguf.cpp"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         # packed-FP32 VALU forms are kept out of every kernel
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def lib_path() -> str:
    return os.path.join(OUT, "liboxb_hip.so")


def build(verbose: bool = False) -> str:
    os.makedirs(OUT, exist_ok=True)
    objs = []

    def compile_one(src: str) -> str:
        obj = os.path.join(OUT, os.path.splitext(src)[0] + ".o")
        cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if src.endswith(".cpp"):
            cmd = [HIPCC, "-x", "hip", *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        msgs = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                         if "packed-fp32-ops" not in l and l.strip())
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{msgs}")
        if msgs and verbose:
            print(msgs, flush=True)
        return obj

    with ThreadPoolExecutor(max_workers=6) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    so = lib_path()
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", so, *objs])
    a = os.path.join(OUT, "liboxb_hip.a")
    if os.path.exists(a):
        os.remove(a)
    subprocess.check_call(["ar", "rcs", a, *objs])
    return so


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
