"""Builds libwekua_hip.so (HIP kernels + C ABI) and libwekua_host.so (the host-side mirror
of wekua's Zig API, used by the Python binding) in-tree with hipcc for gfx950."""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
INCLUDE = os.path.join(ROOT, "include")
OBJ = os.path.join(PKG, "build")

LIB_HIP = os.path.join(PKG, "libwekua_hip.so")
LIB_HOST = os.path.join(PKG, "libwekua_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops off: the compiler must not form v_pk_*_f32 from scalar float code.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
    "-I" + INCLUDE, "-I" + CSRC,
]

HIP_SOURCES = ["wk_runtime.hip", "wk_axpy.hip", "wk_gemm.hip", "wk_gemm_generic.hip", "wk_gemm_mfma.hip", "wk_gemm_dma.hip", "wk_gemm_dma_f64.hip", "wk_gemm_imfma.hip", "wk_gemm_ipack.hip", "wk_gemm_i64pack.hip", "wk_gemm_cpack.hip", "wk_gemm_thin.hip", "wk_gemm_skinny.hip", "wk_nn.hip", "wk_tensor_ops.hip"]


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), res.stdout))
    return res.stdout


def _stale(obj: str, src: str) -> bool:
    """True when `obj` is older than its source or than any header it may include."""
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src] + [os.path.join(d, f) for d in (CSRC, INCLUDE) for f in os.listdir(d) if f.endswith((".hpp", ".h", ".inc"))]
    return any(os.path.getmtime(d) > t for d in deps)


def build_hip(verbose: bool = False, extra_flags=(), incremental: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    jobs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(HIP_SOURCES))) as pool:
        for src in HIP_SOURCES:
            obj = os.path.join(OBJ, src.replace(".hip", ".o"))
            objs.append(obj)
            if incremental and not _stale(obj, os.path.join(CSRC, src)):
                continue
            cmd = [HIPCC] + HIP_FLAGS + list(extra_flags) + ["-c", os.path.join(CSRC, src), "-o", obj]
            jobs.append(pool.submit(_run, cmd))
        for j in jobs:
            out = j.result()
            if verbose and out.strip():
                print(out)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_HIP] + objs)
    return LIB_HIP


def build_host(verbose: bool = False) -> str:
    src = os.path.join(HOST, "wekua_c.cpp")
    if not os.path.exists(src):
        return ""
    cmd = ["g++", "-O2", "-std=c++20", "-fPIC", "-shared", "-Wall", "-Wextra", "-I" + INCLUDE, "-I" + HOST,
           src, "-o", LIB_HOST, "-L" + PKG, "-lwekua_hip", "-Wl,-rpath,$ORIGIN"]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return LIB_HOST


def build_example(verbose: bool = False) -> str:
    """The C++ programs on the host mirror: the usage example (benchmark/gemm.zig's flow) and the reference
    benchmark's size sweeps; built every time to keep them compiling."""
    exe = ""
    for name in ("example_gemm", "benchmark_sweep"):
        src = os.path.join(HOST, name + ".cpp")
        if not os.path.exists(src):
            continue
        exe = os.path.join(OBJ, name)
        out = _run(["g++", "-O2", "-std=c++20", "-Wall", "-Wextra", "-I" + INCLUDE, "-I" + HOST, src, "-o", exe,
                    "-L" + PKG, "-lwekua_hip", "-Wl,-rpath," + PKG])
        if verbose and out.strip():
            print(out)
    return exe


def build_all(verbose: bool = False, incremental: bool = False):
    build_hip(verbose, incremental=incremental)
    build_host(verbose)
    build_example(verbose)


if __name__ == "__main__":
    build_all(verbose=True, incremental="--incremental" in sys.argv)
    print("built", LIB_HIP, LIB_HOST if os.path.exists(LIB_HOST) else "")
