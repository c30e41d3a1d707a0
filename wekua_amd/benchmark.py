"""Counterpart of the reference's `zig build benchmark` (benchmark/{main,gemm,axpy}.zig) for the
HIP path: a table of GEMM times over square sizes and the four transpose pairs, and of AXPY
times over 1-D sizes, on GPU 0.

    python -m wekua_amd.benchmark gemm [--dtype f32] [--sizes 1024 2048 ...] [--variant NAME]
    python -m wekua_amd.benchmark axpy [--dtype f32]
    python -m wekua_amd.benchmark configs        # every BASELINE configuration, one line each

Unlike the reference's harness the inputs are seeded (wekua_amd.synth), times come from
events on the kernel's stream, and every line also gives the rate (TFLOP/s or GB/s).
"""
from __future__ import annotations

import argparse
import sys

import numpy as np

from . import raw, synth

OPS = [(0, 0, "NN"), (0, 1, "NT"), (1, 0, "TN"), (1, 1, "TT")]


def _operand(rd, shape, seed):
    if rd.kind == "f":
        return synth.uniform(seed, shape, rd)
    return synth.integers(seed, shape, rd, -100, 100)


def time_gemm(dev, dtype, M, N, K, op_a, op_b, alpha, beta, iters=10, warmup=2):
    rd = raw.real_np_dtype(dtype)
    a = _operand(rd, (K, M) if op_a else (M, K), 1)
    b = _operand(rd, (N, K) if op_b else (K, N), 2)
    c = _operand(rd, (M, N), 3)
    dA, dB, dC = dev.upload(a), dev.upload(b), dev.upload(c)
    call = lambda: dev.gemm(dtype, op_a, op_b, M, N, K, alpha, dA, a.shape[1], dB, b.shape[1], beta, dC, N)
    for _ in range(warmup):
        call()
    dev.sync()
    ms = dev.time_stream_ms(call, iters)
    variant = dev.lib.wk_gemm_variant(raw.dtype_id(dtype), op_a, op_b, M, N, K, a.shape[1], b.shape[1], N,
                                      dA.ptr, dB.ptr, dC.ptr).decode()
    for d in (dA, dB, dC):
        d.free()
    return ms, variant


def time_axpy(dev, dtype, n, iters=50, warmup=3):
    rd = raw.real_np_dtype(dtype)
    x, y = _operand(rd, (n,), 1), _operand(rd, (n,), 2)
    dx, dy = dev.upload(x), dev.upload(y)
    call = lambda: dev.axpy(dtype, (1, 1, n), dx, n, n, 0.75 if rd.kind == "f" else 3, dy, n, n)
    for _ in range(warmup):
        call()
    dev.sync()
    ms = dev.time_stream_ms(call, iters)
    dx.free()
    dy.free()
    return ms


def cmd_gemm(dev, args):
    print(f"{'dtype':5s} {'n':>6s} {'op':2s} {'ms':>9s} {'TFLOP/s':>9s}  kernel")
    for n in args.sizes:
        for op_a, op_b, name in OPS:
            ms, variant = time_gemm(dev, args.dtype, n, n, n, op_a, op_b, 1.5 if args.dtype[0] == "f" else 3,
                                    0.5 if args.dtype[0] == "f" else 2)
            print(f"{args.dtype:5s} {n:6d} {name:2s} {ms:9.4f} {2.0 * n ** 3 / ms / 1e9:9.2f}  {variant}", flush=True)


def cmd_axpy(dev, args):
    print(f"{'dtype':5s} {'n':>10s} {'us':>9s} {'GB/s':>8s}")
    for lg in range(12, 29):
        n = 1 << lg
        ms = time_axpy(dev, args.dtype, n)
        nbytes = 3 * n * raw.elem_size(args.dtype)
        print(f"{args.dtype:5s} {n:10d} {ms * 1e3:9.2f} {nbytes / ms / 1e6:8.0f}", flush=True)


def cmd_configs(dev, args):
    rows = []
    ms, v = time_gemm(dev, "f32", 512, 512, 512, 0, 0, 1.0, 0.0)
    rows.append(("1 f32 512^3 NN a=1 b=0", ms, 2 * 512 ** 3 / ms / 1e9, "TFLOP/s", v))
    for dt in ("f32", "f64"):
        for lg in (20, 24, 28):
            ms = time_axpy(dev, dt, 1 << lg)
            rows.append((f"2 axpy {dt} n=2^{lg}", ms, 3 * (1 << lg) * raw.elem_size(dt) / ms / 1e6, "GB/s", "axpy_stream"))
    for n in (1024, 2048, 4096, 8192):
        for op_a, op_b, name in OPS:
            ms, v = time_gemm(dev, "f32", n, n, n, op_a, op_b, 1.5, 0.5)
            rows.append((f"3 f32 {n}^3 {name}", ms, 2.0 * n ** 3 / ms / 1e9, "TFLOP/s", v))
    for (M, N, K) in ((1000, 1000, 1000), (4097, 4095, 4093)):
        for op_a, op_b, name in OPS:
            ms, v = time_gemm(dev, "f32", M, N, K, op_a, op_b, 1.5, 0.5)
            rows.append((f"3 f32 {M}x{N}x{K} {name}", ms, 2.0 * M * N * K / ms / 1e9, "TFLOP/s", v))
    ms, v = time_gemm(dev, "f64", 4096, 4096, 4096, 0, 0, 1.0, 1.0)
    rows.append(("4 f64 4096^3 NN", ms, 2.0 * 4096 ** 3 / ms / 1e9, "TFLOP/s", v))
    ms, v = time_gemm(dev, "f64", 8192, 256, 8192, 0, 0, 1.0, 1.0)
    rows.append(("4 f64 8192x256x8192 NN", ms, 2.0 * 8192 * 256 * 8192 / ms / 1e9, "TFLOP/s", v))
    ms, v = time_gemm(dev, "i32", 2048, 2048, 2048, 0, 0, 3, -2)
    rows.append(("4 i32 2048^3 NN", ms, 2.0 * 2048 ** 3 / ms / 1e9, "TOP/s", v))
    print(f"{'config':34s} {'ms':>9s} {'rate':>9s} unit     kernel")
    for name, ms, rate, unit, v in rows:
        print(f"{name:34s} {ms:9.4f} {rate:9.2f} {unit:8s} {v}")


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m wekua_amd.benchmark")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("gemm")
    g.add_argument("--dtype", default="f32")
    g.add_argument("--sizes", type=int, nargs="+", default=[4 << i for i in range(4, 12)])
    g.add_argument("--variant", default="auto")
    a = sub.add_parser("axpy")
    a.add_argument("--dtype", default="f32")
    c = sub.add_parser("configs")
    c.add_argument("--variant", default="auto")
    args = ap.parse_args(argv)
    dev = raw.Device(0)
    try:
        if getattr(args, "variant", "auto") != "auto":
            raw.check(dev.lib.wk_gemm_force_variant(args.variant.encode()), "wk_gemm_force_variant")
        {"gemm": cmd_gemm, "axpy": cmd_axpy, "configs": cmd_configs}[args.cmd](dev, args)
    finally:
        dev.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
