#!/usr/bin/env python3
"""Benchmark of the BLAS hot path on one MI355X.

A "step" is one call of the headline workload: f32 GEMM C = 1.5*A*B + 0.5*C at
M = N = K = 8192 (no transposes), operands resident in HBM.  The AXPY half of the metric
(y = 0.75*x + y, f32, n = 2^28) is measured in the same run and reported beside it.

Prints ONE JSON line:  metric/value/unit as BASELINE.json names them, `roofline` for the
GEMM kernel (MFMA-bound), `axpy` with its own HBM roofline, and `cpu_baseline`: the
reference-order CPU restatement (oracle/) timed on this box's host cores on a bounded
sample of the same GEMM.  The oracle is used here only as that timed baseline.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

F32_MATRIX_PEAK_TFLOPS = 157.3   # MI355X dense f32 matrix peak
HBM_PEAK_GBS = 8000.0            # MI355X HBM3E


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def read_traffic(name: str):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE), if recorded."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(name)
    except (OSError, ValueError):
        return None


def gemm_leg(wk, synth, n, steps, warmup):
    """The headline call through the reference-shaped API: Tensor.alloc + memory.readFromBuffer, then
    `steps` calls of blas.gemm(pipeline, 1.5, A, N, B, N, 0.5, C, null) on one pipeline."""
    rd = np.float32
    t0 = time.time()
    a = synth.uniform(synth.config_seed(3, 0), (n, n), rd)
    b = synth.uniform(synth.config_seed(3, 1), (n, n), rd)
    c = synth.uniform(synth.config_seed(3, 2), (n, n), rd)
    ctx = wk.Context.initFromDeviceType(wk.DeviceType.all)
    pipeline = wk.Pipeline.init(ctx.command_queues[0])
    A = wk.Tensor.alloc("f32", ctx, pipeline, (n, n))
    B = wk.Tensor.alloc("f32", ctx, pipeline, (n, n))
    C = wk.Tensor.alloc("f32", ctx, pipeline, (n, n))
    for t, h in ((A, a), (B, b), (C, c)):
        wk.memory.readFromBuffer(pipeline, t, h)
    pipeline.waitAndCleanup()
    log(f"[bench] gemm operands {n}x{n} f32 generated + uploaded in {time.time() - t0:.1f}s "
        f"(row pitch {A.row_pitch} elements)")
    lib = wk._capi.load()
    variant = lib.wk_gemm_variant(wk.dtype_id("f32"), 0, 0, n, n, n, A.row_pitch, B.row_pitch, C.row_pitch,
                                  A.buffer, B.buffer, C.buffer).decode()
    N_ = wk.blas.Operation.no_transpose

    def step():
        wk.blas.gemm(pipeline, 1.5, A, N_, B, N_, 0.5, C, None)

    for _ in range(warmup):
        step()
    pipeline.waitAndCleanup()
    # timed region: exactly `steps` calls.  Wall clock (sync on both sides) gives `value`; events
    # recorded on the pipeline's own stream around the same launches give the kernel time.
    stream = wk._lib().wkz_context_stream(ctx._h, 0)
    device = wk._lib().wkz_context_device(ctx._h)
    import ctypes
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    wk._capi.check(lib.wk_event_create(device, ctypes.byref(e0)))
    wk._capi.check(lib.wk_event_create(device, ctypes.byref(e1)))
    t0 = time.perf_counter()
    wk._capi.check(lib.wk_event_record(e0, stream))
    for _ in range(steps):
        step()
    wk._capi.check(lib.wk_event_record(e1, stream))
    pipeline.waitAndCleanup()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = ctypes.c_float()
    wk._capi.check(lib.wk_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
    kernel_ms = ms.value / steps
    lib.wk_event_destroy(e0)
    lib.wk_event_destroy(e1)
    flops = 2.0 * n * n * n
    for t in (A, B, C):
        t.release(pipeline)
    pipeline.deinit()
    ctx.deinit()
    return {
        "variant": variant, "wall_ms": wall_ms, "kernel_ms": kernel_ms,
        "tflops_wall": flops / wall_ms / 1e9, "tflops_kernel": flops / kernel_ms / 1e9,
        "a": a, "b": b,
    }


def axpy_leg(dev, raw, synth, dtype, log2n, steps, warmup):
    rd = raw.real_np_dtype(dtype)
    n = 1 << log2n
    x = synth.uniform(synth.config_seed(2, 0), (n,), rd)
    y = synth.uniform(synth.config_seed(2, 1), (n,), rd)
    dx, dy = dev.upload(x), dev.upload(y)

    def step():
        dev.axpy(dtype, (1, 1, n), dx, n, n, 0.75, dy, n, n)

    for _ in range(warmup):
        step()
    dev.sync()
    ms = dev.time_stream_ms(step, steps)
    dx.free()
    dy.free()
    nbytes = 3.0 * n * rd.itemsize
    return {"dtype": dtype, "n": n, "us": ms * 1e3, "gbs": nbytes / ms / 1e6, "bytes": nbytes}


def cpu_baseline_leg(a, b, rows, threads):
    """The reference CPU device's algorithm (packed path, block 16, 8 f32 lanes) on the first
    `rows` rows of the same 8192^3 product, timed on this host."""
    import oracle
    n = a.shape[1]
    a_s = np.ascontiguousarray(a[:rows])
    c_s = np.zeros((rows, n), dtype=np.float32)
    t0 = time.perf_counter()
    oracle.gemm("f32", 1.5, a_s, 0, b, 0, 0.5, c_s, vector_width=8, packed=True, threads=threads)
    dt = time.perf_counter() - t0
    return {"seconds": dt, "tflops": 2.0 * rows * n * n / dt / 1e12}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--n", type=int, default=8192, help="square GEMM size (default: the headline 8192)")
    ap.add_argument("--axpy-log2n", type=int, default=28)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=8192)
    ap.add_argument("--no-mlp", action="store_true", help="skip the MLP training step leg (BASELINE configuration 5)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch the plain 1 GiB copy kernel a few times, so that a profiler run of this "
                         "command holds a kernel of known HBM traffic to scale byte counters against")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build uses one GPU; --gpus N with N > 1 is not supported "
              "(GEMM and AXPY shard over GPUs without any exchange step: every GPU would run this same benchmark on its share)", file=sys.stderr)
        sys.exit(2)

    import wekua_amd as wk                # fails loudly if the native libraries are missing
    from wekua_amd import raw, synth

    g = gemm_leg(wk, synth, args.n, args.steps, args.warmup)
    dev = raw.Device(0)
    props = dev.props()
    log(f"[bench] device: {props.name.decode()} {props.arch.decode()} CUs={props.compute_units}")
    log(f"[bench] gemm f32 {args.n}^3 [{g['variant']}]: {g['kernel_ms']:.3f} ms/launch (events), "
        f"{g['wall_ms']:.3f} ms/step (wall) -> {g['tflops_kernel']:.1f} TFLOP/s")

    ax = axpy_leg(dev, raw, synth, "f32", args.axpy_log2n, max(args.steps, 20), args.warmup)
    ax64 = axpy_leg(dev, raw, synth, "f64", args.axpy_log2n, max(args.steps, 20), args.warmup)
    log(f"[bench] axpy f32 2^{args.axpy_log2n}: {ax['us']:.1f} us -> {ax['gbs']:.0f} GB/s; "
        f"f64: {ax64['us']:.1f} us -> {ax64['gbs']:.0f} GB/s")
    if args.calibrate:
        nbytes = 1 << 30
        src, dst = dev.malloc(nbytes), dev.malloc(nbytes)
        from wekua_amd._capi import check
        check(dev.lib.wk_memset_async(dev.stream, src.ptr, 1, nbytes), "memset")
        ms = dev.time_stream_ms(lambda: check(dev.lib.wk_copy_kernel(dev.stream, dst.ptr, src.ptr, nbytes), "copy"), 5)
        log(f"[bench] calibration copy 1 GiB: {ms * 1e3:.1f} us -> {2 * nbytes / ms / 1e6:.0f} GB/s (read + write)")
        src.free()
        dst.free()
    dev.close()

    mlp = None
    if not args.no_mlp:
        from wekua_amd import benchmark
        m = benchmark.time_mlp_step(steps=max(args.steps, 10), warmup=args.warmup)
        log(f"[bench] mlp step 1024-4096-4096-1024 f32 batch 2048 adam: {m['stream_ms']:.3f} ms/step "
            f"-> {m['tflops']:.1f} TFLOP/s over its GEMM flops")
        mlp = {"workload": "MLP training step 1024-4096-4096-1024, f32, batch 2048, tanh/tanh/sigmoid, MSE, Adam lr=1e-3 "
                           "(BASELINE config 5): forward + loss + backward + update",
               "ms_per_step": m["stream_ms"], "wall_ms_per_step": m["wall_ms"], "gemm_flops_per_step": m["flops"],
               "value": m["tflops"], "unit": "TFLOP/s", "frac_of_f32_matrix_peak": m["tflops"] / F32_MATRIX_PEAK_TFLOPS}

    other = None
    if not args.no_mlp:   # the remaining benchmark configurations, a few launches each
        from wekua_amd import benchmark
        ses = benchmark.Session()
        try:
            other = {}
            for key, dtype, (M, N, K), alpha, beta, unit in (("f64_gemm_4096", "f64", (4096, 4096, 4096), 1.0, 1.0, "TFLOP/s"),
                                                             ("f64_gemm_8192x256x8192", "f64", (8192, 256, 8192), 1.0, 1.0, "TFLOP/s"),
                                                             ("i32_gemm_2048", "i32", (2048, 2048, 2048), 3, -2, "TOP/s"),
                                                             ("f32_gemm_1000", "f32", (1000, 1000, 1000), 1.5, 0.5, "TFLOP/s"),
                                                             ("f32_gemm_4097x4095x4093", "f32", (4097, 4095, 4093), 1.5, 0.5, "TFLOP/s")):
                ms, variant = benchmark.time_gemm(ses, dtype, M, N, K, 0, 0, alpha, beta)
                other[key] = {"ms": ms, "value": 2.0 * M * N * K / ms / 1e9, "unit": unit, "kernel": variant}
                log(f"[bench] {key}: {ms:.4f} ms -> {other[key]['value']:.1f} {unit} [{variant}]")
        finally:
            ses.close()

    cpu = None
    if not args.no_cpu_baseline:
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16), 16)
        rows = min(args.cpu_rows, args.n)
        log(f"[bench] cpu baseline: reference-order restatement, {rows} of {args.n} rows, {cores} threads ...")
        c = cpu_baseline_leg(g["a"], g["b"], rows, cores)
        log(f"[bench] cpu baseline: {c['seconds']:.1f}s -> {c['tflops'] * 1e3:.1f} GFLOP/s")
        cpu = {
            "value": c["tflops"], "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"rows 0..{rows - 1} of the same {args.n}^3 f32 GEMM ({rows}x{args.n}x{args.n}), "
                      "reference CPU-device algorithm (packed path, block 16, 8 lanes), one call",
        }

    flops = 2.0 * args.n ** 3
    out = {
        "metric": "f32 GEMM TFLOP/s @8192^3 + AXPY HBM GB/s, each as % of MI355X roofline",
        "value": g["tflops_wall"], "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": g["wall_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"f32 GEMM C=1.5*A*B+0.5*C, M=N=K={args.n}, no transposes, uniform[-1,1) seeded "
                               f"(BASELINE config 3 headline shape); plus AXPY y=0.75*x+y n=2^{args.axpy_log2n}",
                   "kernel": g["variant"]},
        "roofline": {"bound": "mfma", "achieved": g["tflops_kernel"], "peak": F32_MATRIX_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": g["tflops_kernel"] / F32_MATRIX_PEAK_TFLOPS,
                     "traffic": read_traffic("gemm_f32_8192"), "flops_per_launch": flops,
                     "kernel_ms": g["kernel_ms"]},
        "axpy": {"value": ax["gbs"], "unit": "GB/s", "dtype": "f32", "n": ax["n"], "us_per_call": ax["us"],
                 "roofline": {"bound": "hbm", "achieved": ax["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": ax["gbs"] / HBM_PEAK_GBS, "traffic": read_traffic("axpy_f32_2p28"),
                              "bytes_per_launch": ax["bytes"]},
                 "f64": {"value": ax64["gbs"], "us_per_call": ax64["us"], "frac": ax64["gbs"] / HBM_PEAK_GBS}},
        "mlp_step": mlp,
        "configs": other,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
