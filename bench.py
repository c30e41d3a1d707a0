#!/usr/bin/env python3
"""Benchmark of the BLAS hot path on one MI355X.

A "step" is one call of the headline workload: f32 GEMM C = 1.5*A*B + 0.5*C at
M = N = K = 8192 (no transposes), operands resident in HBM.  The AXPY half of the metric
(y = 0.75*x + y, f32, n = 2^28) is measured in the same run and reported beside it.

Prints ONE JSON line:
  metric / value / unit   as the benchmark definition names them (the headline GEMM, wall clock);
  roofline                the headline GEMM kernel against the f32 matrix peak, from events on its stream;
  axpy                    f32 / f64 at n = 2^28 against the HBM peak, the same kernel under two placements
                          of x and y (same offset inside a 4 KiB block; y 3 KiB further in), and the CPU
                          baseline for every AXPY size;
  configs                 every GEMM and AXPY benchmark configuration (512^3; 1024..8192^3 x NN/NT/TN/TT;
                          1000^3 and 4097x4095x4093 x 4; f64 4096^3 and 8192x256x8192; int32 2048^3; AXPY
                          2^20 / 2^24 / 2^28 x f32 / f64), each with its own roofline fraction;
  mlp_step                the MLP training step;
  cpu_baseline            the reference-order CPU restatement (oracle/) timed on this box's host cores
                          on the headline GEMM; `cpu_baselines` holds the other shapes it was timed on;
  perf_floor              the two rates a regression must not pass unnoticed; the exit status is 3 when
                          one is missed (the JSON line is printed either way; --no-floor disables it).
The oracle is used here only as that timed baseline.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

F32_MATRIX_PEAK_TFLOPS = 157.3   # MI355X dense f32 matrix peak
HBM_PEAK_GBS = 8000.0            # MI355X HBM3E
FLOOR_GEMM_TFLOPS = 130.0        # f32 8192^3 NN (measured 139-144 across boxes)
FLOOR_AXPY_GBS = 6600.0          # f32 n = 2^28 (measured 6820-6860 across boxes)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def read_traffic(name: str, kernel: str):
    """HBM bytes per launch recorded from a rocprofv3 --pmc run (FETCH_SIZE / WRITE_SIZE) of this
    command; not measured in this run.  Returns (bytes, stale): stale when the record was taken on
    another kernel than the one this run launches."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f).get(name)
    except (OSError, ValueError):
        return None, None
    if not isinstance(rec, dict):
        return None, None
    return rec.get("bytes"), rec.get("kernel") != kernel


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


def axpy_placement_leg(dev, raw, dtype, log2n, steps, warmup):
    """wk_axpy at n = 2^log2n on operands placed by hand inside two device blocks: x at the start of
    a 4 KiB block, y once at the same offset inside its own (where two fresh device allocations put
    them) and once 3 KiB further in (what the library's allocator gives neighbours in allocation
    order).  Same kernel, same data; only the distance between the base addresses differs."""
    rd = raw.real_np_dtype(dtype)
    n = 1 << log2n
    nbytes = n * rd.itemsize
    bx, by = dev.malloc(nbytes + 16384), dev.malloc(nbytes + 16384)
    up = lambda p: (p + 4095) // 4096 * 4096
    x0, y0 = up(bx.ptr.value), up(by.ptr.value)
    did = raw.dtype_id(dtype)
    s3 = (ctypes.c_uint64 * 3)(1, 1, n)
    lo, span = raw.scalar_bytes(dtype, -1.0), raw.scalar_bytes(dtype, 2.0)
    for seed, p in ((21, x0), (22, y0)):
        raw.check(dev.lib.wk_random_uniform(dev.stream, did, (ctypes.c_uint64 * 3)(1, 1, n + 3072 // rd.itemsize),
                                            ctypes.c_void_p(p), n + 3072 // rd.itemsize, n + 3072 // rd.itemsize, seed,
                                            ctypes.cast(lo, ctypes.c_void_p), ctypes.cast(span, ctypes.c_void_p)),
                  "wk_random_uniform")
    alpha = raw.scalar_bytes(dtype, 0.75)
    out = {}
    for name, yp in (("same_offset_in_4KiB", y0), ("y_plus_3KiB", y0 + 3072)):
        def step():
            raw.check(dev.lib.wk_axpy(dev.stream, did, s3, ctypes.c_void_p(x0), n, n, ctypes.c_void_p(yp), n, n,
                                      ctypes.cast(alpha, ctypes.c_void_p)), "wk_axpy")
        for _ in range(warmup):
            step()
        dev.sync()
        ms = dev.time_stream_ms(step, steps)
        out[name] = 3.0 * nbytes / ms / 1e6
    bx.free()
    by.free()
    return out


def memory_ceilings(dev, raw, log2n):
    """What the memory system gives simpler access patterns on this box in this run, for scale next to
    the AXPY figure (2 read streams + 1 write stream).  Three probes in the AXPY kernel's own shape (one
    wavefront per work-group, one 16-byte vector per lane, non-temporal loads, streaming stores): a copy
    (1 read + 1 write stream), one read stream and two read streams; and the plain grid-stride copy kernel
    that calibrates the profiler's byte counters.  n = 2^log2n f32 of random data in [-1, 1); median of
    five batches of ten launches each."""
    from wekua_amd._capi import check
    n = 1 << log2n
    nbytes = 4 * n
    src, dst = dev.malloc(nbytes), dev.malloc(nbytes)
    did = raw.dtype_id("f32")
    s3 = (ctypes.c_uint64 * 3)(1, 1, n)
    lo, span = raw.scalar_bytes("f32", -1.0), raw.scalar_bytes("f32", 2.0)
    for buf, seed in ((src, 5), (dst, 6)):
        check(dev.lib.wk_random_uniform(dev.stream, did, s3, buf.ptr, n, n, seed, ctypes.cast(lo, ctypes.c_void_p),
                                        ctypes.cast(span, ctypes.c_void_p)), "wk_random_uniform")
    # 0x7fc01234 is a NaN as f32: neither a value in [-1, 1) nor, in all four words, the xor of two of them
    sentinel = 0x7fc01234
    median = lambda call: sorted(dev.time_stream_ms(call, 10) for _ in range(5))[2]
    probe = lambda kind: (lambda: check(dev.lib.wk_stream_probe(dev.stream, kind, dst.ptr, src.ptr, nbytes, sentinel), "probe"))
    plain = lambda: check(dev.lib.wk_copy_kernel(dev.stream, dst.ptr, src.ptr, nbytes), "copy")
    for call in (probe(0), probe(1), probe(2), plain):
        call()
    dev.sync()
    ms = {"copy": median(probe(0)), "read": median(probe(1)), "read2": median(probe(2)), "plain": median(plain)}
    for b in (src, dst):
        b.free()
    return {"copy_GBs": 2.0 * nbytes / ms["copy"] / 1e6, "read_GBs": nbytes / ms["read"] / 1e6,
            "two_reads_GBs": 2.0 * nbytes / ms["read2"] / 1e6, "plain_copy_GBs": 2.0 * nbytes / ms["plain"] / 1e6,
            "n": n, "dtype": "f32",
            "what": "probes in the AXPY kernel's shape: copy (1 read + 1 write stream), read (1 read stream), two_reads "
                    "(2 read streams); plain_copy is the grid-stride copy kernel that calibrates the byte counters; "
                    "bytes moved / time, median of 5 batches of 10 launches"}


def cpu_gemm_leg(dtype, M, N, K, alpha, beta, threads, a=None, b=None):
    """The reference CPU device's algorithm (packed path, block 16, 8 lanes for f32) timed on this host."""
    import oracle
    from wekua_amd import synth
    rd = oracle.real_np_dtype(dtype)
    if a is None:
        if rd.kind == "f":
            a, b = synth.uniform(1, (M, K), rd), synth.uniform(2, (K, N), rd)
        else:
            a, b = synth.integers(1, (M, K), rd, -100, 100), synth.integers(2, (K, N), rd, -100, 100)
    c = np.zeros((M, N), dtype=rd)
    t0 = time.perf_counter()
    oracle.gemm(dtype, alpha, a, 0, b, 0, beta, c, vector_width=8, packed=True, threads=threads)
    dt = time.perf_counter() - t0
    return {"seconds": dt, "rate": 2.0 * M * N * K / dt / 1e12}


def cpu_axpy_leg(dtype, log2n, threads, reps):
    """axpy.cl's element-wise kernel with its work-items spread over the host threads, in place."""
    import oracle
    rd = oracle.real_np_dtype(dtype)
    n = 1 << log2n
    rng = np.random.default_rng(log2n)
    x = rng.random(n, dtype=rd) * 2 - 1
    y = rng.random(n, dtype=rd) * 2 - 1
    oracle.axpy_inplace(dtype, x, 0.75, y, contract=True, threads=threads)   # first touch, thread start-up
    t0 = time.perf_counter()
    for _ in range(reps):
        oracle.axpy_inplace(dtype, x, 0.75, y, contract=True, threads=threads)
    dt = (time.perf_counter() - t0) / reps
    return {"seconds": dt, "gbs": 3.0 * n * rd.itemsize / dt / 1e9}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--n", type=int, default=8192, help="square GEMM size (default: the headline 8192)")
    ap.add_argument("--axpy-log2n", type=int, default=28)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=8192)
    ap.add_argument("--no-mlp", action="store_true", help="skip the MLP training step leg (benchmark configuration 5)")
    ap.add_argument("--no-configs", action="store_true", help="skip the sweep over the other benchmark configurations")
    ap.add_argument("--no-floor", action="store_true", help="do not turn a missed performance floor into exit status 3")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build uses one GPU; --gpus N with N > 1 is not supported "
              "(GEMM and AXPY shard over GPUs without any exchange step: every GPU would run this same benchmark on its share)", file=sys.stderr)
        sys.exit(2)

    import wekua_amd as wk                # fails loudly if the native libraries are missing
    from wekua_amd import benchmark, raw, synth

    g = gemm_leg(wk, synth, args.n, args.steps, args.warmup)
    dev = raw.Device(0)
    props = dev.props()
    log(f"[bench] device: {props.name.decode()} {props.arch.decode()} CUs={props.compute_units}")
    log(f"[bench] gemm f32 {args.n}^3 [{g['variant']}]: {g['kernel_ms']:.3f} ms/launch (events), "
        f"{g['wall_ms']:.3f} ms/step (wall) -> {g['tflops_kernel']:.1f} TFLOP/s")

    place = {dt: axpy_placement_leg(dev, raw, dt, args.axpy_log2n, max(args.steps, 20), args.warmup) for dt in ("f32", "f64")}
    for dt in ("f32", "f64"):
        log(f"[bench] axpy {dt} 2^{args.axpy_log2n} by placement of y against x: same offset inside a 4 KiB block "
            f"{place[dt]['same_offset_in_4KiB']:.0f} GB/s, 3 KiB further in {place[dt]['y_plus_3KiB']:.0f} GB/s")
    ceilings = memory_ceilings(dev, raw, args.axpy_log2n)
    log(f"[bench] memory rates on this box in the AXPY kernel's shape: copy (1 read + 1 write stream) {ceilings['copy_GBs']:.0f} GB/s, "
        f"1 read stream {ceilings['read_GBs']:.0f} GB/s, 2 read streams {ceilings['two_reads_GBs']:.0f} GB/s; "
        f"plain grid-stride copy {ceilings['plain_copy_GBs']:.0f} GB/s")
    dev.close()

    # every benchmark configuration through the reference-shaped API (tensors from Tensor.alloc, so with
    # the library's own pitches and placement), operands drawn on the device
    configs = None
    off_sizes = None
    if not args.no_configs:
        ses = benchmark.Session()
        try:
            configs = benchmark.run_baseline_configs(ses, log=lambda m: log("[bench] " + m))
            off_sizes = benchmark.run_off_benchmark_sizes(ses, log=lambda m: log("[bench] " + m))
        finally:
            ses.close()
    ax_key = f"2_axpy_f32_2p{args.axpy_log2n}"
    if configs and ax_key in configs:
        ax_gbs, ax_us = configs[ax_key]["value"], configs[ax_key]["ms"] * 1e3
        ax64 = configs[f"2_axpy_f64_2p{args.axpy_log2n}"]
    else:   # the sweep was skipped: the coloured placement stands for the tensors' own
        ax_gbs = place["f32"]["y_plus_3KiB"]
        ax_us = 3.0 * 4 * (1 << args.axpy_log2n) / ax_gbs / 1e3
        ax64 = {"value": place["f64"]["y_plus_3KiB"], "ms": 3.0 * 8 * (1 << args.axpy_log2n) / place["f64"]["y_plus_3KiB"] / 1e6}

    mlp = None
    if not args.no_mlp:
        m = benchmark.time_mlp_step(steps=max(args.steps, 10), warmup=args.warmup)
        log(f"[bench] mlp step 1024-4096-4096-1024 f32 batch 2048 adam: {m['stream_ms']:.3f} ms/step "
            f"-> {m['tflops']:.1f} TFLOP/s over its GEMM flops")
        mlp = {"workload": "MLP training step 1024-4096-4096-1024, f32, batch 2048, tanh/tanh/sigmoid, MSE, Adam lr=1e-3 "
                           "(benchmark configuration 5): forward + loss + backward + update",
               "ms_per_step": m["stream_ms"], "wall_ms_per_step": m["wall_ms"], "gemm_flops_per_step": m["flops"],
               "value": m["tflops"], "unit": "TFLOP/s",
               "roofline": {"bound": "mfma", "achieved": m["tflops"], "peak": F32_MATRIX_PEAK_TFLOPS, "unit": "TFLOP/s",
                            "frac": m["tflops"] / F32_MATRIX_PEAK_TFLOPS}}

    cpu = None
    cpu_all = None
    axpy_cpu = None
    if not args.no_cpu_baseline:
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16), 16)
        rows = min(args.cpu_rows, args.n)
        log(f"[bench] cpu baseline: reference-order restatement, {rows} of {args.n} rows, {cores} threads ...")
        c = cpu_gemm_leg("f32", rows, args.n, args.n, 1.5, 0.5, cores, np.ascontiguousarray(g["a"][:rows]), g["b"])
        log(f"[bench] cpu baseline: {c['seconds']:.1f}s -> {c['rate'] * 1e3:.1f} GFLOP/s")
        kind = "reference CPU-device algorithm (packed path, block 16, 8 lanes), one call"
        cpu = {
            "value": c["rate"], "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"rows 0..{rows - 1} of the same {args.n}^3 f32 GEMM ({rows}x{args.n}x{args.n}), {kind}",
        }
        cpu_all = {}
        for key, dtype, (M, N, K), alpha, beta, unit in (("1_f32_gemm_512_NN", "f32", (512, 512, 512), 1.0, 0.0, "TFLOP/s"),
                                                         ("3_f32_gemm_1024_NN", "f32", (1024, 1024, 1024), 1.5, 0.5, "TFLOP/s"),
                                                         ("3_f32_gemm_2048_NN", "f32", (2048, 2048, 2048), 1.5, 0.5, "TFLOP/s"),
                                                         ("4_i32_gemm_2048_NN", "i32", (2048, 2048, 2048), 3, -2, "TOP/s")):
            cpu_gemm_leg(dtype, 256, 256, 256, alpha, beta, cores)   # thread start-up outside the timed call
            r = cpu_gemm_leg(dtype, M, N, K, alpha, beta, cores)
            cpu_all[key] = {"value": r["rate"], "unit": unit, "cores": cores, "kind": "port", "seconds": r["seconds"],
                            "sample": f"the whole {M}x{N}x{K} {dtype} GEMM, {kind}"}
            log(f"[bench] cpu baseline {key}: {r['seconds'] * 1e3:.1f} ms -> {r['rate'] * 1e3:.1f} G{unit[1:]}")
        axpy_cpu = {}
        for dt in ("f32", "f64"):
            for lg in (20, 24, args.axpy_log2n):
                r = cpu_axpy_leg(dt, lg, cores, 20 if lg <= 24 else 3)
                axpy_cpu[f"2_axpy_{dt}_2p{lg}"] = {"value": r["gbs"], "unit": "GB/s", "cores": cores, "kind": "port",
                                                   "sample": f"the whole n=2^{lg} {dt} AXPY in place, axpy.cl's element-wise kernel "
                                                             "spread over the host threads"}
                log(f"[bench] cpu baseline axpy {dt} 2^{lg}: {r['seconds'] * 1e3:.2f} ms -> {r['gbs']:.1f} GB/s")
        if configs:
            for k, v in list(cpu_all.items()) + list(axpy_cpu.items()):
                if k in configs:
                    configs[k]["cpu_baseline"] = v

    floor = {"gemm_f32_8192_NN_TFLOPs": {"floor": FLOOR_GEMM_TFLOPS, "value": g["tflops_kernel"]},
             "axpy_f32_2p28_GBs": {"floor": FLOOR_AXPY_GBS, "value": ax_gbs}}
    floor_ok = all(v["value"] >= v["floor"] for v in floor.values()) or args.n != 8192 or args.axpy_log2n != 28
    floor["ok"] = bool(floor_ok)

    flops = 2.0 * args.n ** 3
    gemm_traffic, gemm_traffic_stale = read_traffic("gemm_f32_8192", g["variant"]) if args.n == 8192 else (None, None)
    axpy_traffic, axpy_traffic_stale = read_traffic("axpy_f32_2p28", "axpy_stream") if args.axpy_log2n == 28 else (None, None)
    out = {
        "metric": "f32 GEMM TFLOP/s @8192^3 + AXPY HBM GB/s, each as % of MI355X roofline",
        "value": g["tflops_wall"], "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": g["wall_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"f32 GEMM C=1.5*A*B+0.5*C, M=N=K={args.n}, no transposes, uniform[-1,1) seeded "
                               f"(benchmark configuration 3, headline shape); plus AXPY y=0.75*x+y n=2^{args.axpy_log2n}",
                   "kernel": g["variant"]},
        "roofline": {"bound": "mfma", "achieved": g["tflops_kernel"], "peak": F32_MATRIX_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": g["tflops_kernel"] / F32_MATRIX_PEAK_TFLOPS,
                     "traffic": gemm_traffic, "traffic_stale": gemm_traffic_stale,
                     "traffic_source": "recorded from profiles/traffic.json, not measured in this run",
                     "flops_per_launch": flops, "kernel_ms": g["kernel_ms"]},
        "axpy": {"value": ax_gbs, "unit": "GB/s", "dtype": "f32", "n": 1 << args.axpy_log2n, "us_per_call": ax_us,
                 "roofline": {"bound": "hbm", "achieved": ax_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": ax_gbs / HBM_PEAK_GBS, "traffic": axpy_traffic, "traffic_stale": axpy_traffic_stale,
                              "traffic_source": "recorded from profiles/traffic.json, not measured in this run",
                              "bytes_per_launch": 3.0 * 4 * (1 << args.axpy_log2n)},
                 "f64": {"value": ax64["value"], "us_per_call": ax64["ms"] * 1e3, "frac": ax64["value"] / HBM_PEAK_GBS},
                 "over_batches": (configs or {}).get(ax_key, {}).get("over_batches"),
                 "f64_over_batches": (configs or {}).get(f"2_axpy_f64_2p{args.axpy_log2n}", {}).get("over_batches"),
                 "ceilings": ceilings,
                 "placement_GBs": place,
                 "cpu_baseline": (axpy_cpu or {}).get(f"2_axpy_f32_2p{args.axpy_log2n}")},
        "mlp_step": mlp,
        "configs": configs,
        "off_benchmark_sizes": off_sizes,
        "cpu_baseline": cpu,
        "cpu_baselines": cpu_all,
        "perf_floor": floor,
    }
    print(json.dumps(out), flush=True)
    if not floor_ok and not args.no_floor:
        log(f"[bench] below the performance floor: {floor}")
        sys.exit(3)


if __name__ == "__main__":
    main()
