"""Counterpart of the reference's `zig build benchmark` (benchmark/{main,gemm,axpy}.zig) for the
HIP path: a table of GEMM times over square sizes and the four transpose pairs, and of AXPY
times over 1-D sizes, on GPU 0.

    python -m wekua_amd.benchmark gemm [--dtype f32] [--sizes 1024 2048 ...] [--shapes 8192x256x8192 ...] [--ops NN TN] [--variant NAME]
    python -m wekua_amd.benchmark axpy [--dtype f32]
    python -m wekua_amd.benchmark configs        # every GEMM / AXPY benchmark configuration, one line each
    python -m wekua_amd.benchmark tensor         # transpose / copy / random.uniform / toComplex streaming rates
    python -m wekua_amd.benchmark probe          # cost of an empty and of a store-only launch on the GEMM grids
    python -m wekua_amd.benchmark mlp [--dtype f32] [--sizes 1024 4096 4096 1024] [--batch 2048] [--optimizer adam]

Everything goes through the reference-shaped API (Tensor.alloc, memory.readFromBuffer, blas.*).
Unlike the reference's harness the inputs are seeded (wekua_amd.synth), times come from
events on the pipeline's stream after a warm-up by time, and every line also gives the rate
(TFLOP/s or GB/s).
"""
from __future__ import annotations

import argparse
import sys

import numpy as np

from . import raw, synth

OPS = [(0, 0, "NN"), (0, 1, "NT"), (1, 0, "TN"), (1, 1, "TT")]


def _operand(rd, shape, seed, full_range=False):
    if rd.kind == "f":
        return synth.uniform(seed, shape, rd)
    if full_range:
        info = np.iinfo(rd)
        return synth.integers(seed, shape, rd, int(info.min), int(info.max))
    return synth.integers(seed, shape, rd, -100, 100)


class Session:
    """One Context + Pipeline and the event pair used to time launches on the pipeline's stream."""

    def __init__(self):
        import ctypes

        import wekua_amd as wk
        self.wk, self.ct = wk, ctypes
        self.ctx = wk.Context.initFromDeviceType(wk.DeviceType.all)
        self.pipeline = wk.Pipeline.init(self.ctx.command_queues[0])
        self.lib = wk._capi.load()
        self.stream = wk._lib().wkz_context_stream(self.ctx._h, 0)
        device = wk._lib().wkz_context_device(self.ctx._h)
        self.e0, self.e1 = ctypes.c_void_p(), ctypes.c_void_p()
        wk._capi.check(self.lib.wk_event_create(device, ctypes.byref(self.e0)))
        wk._capi.check(self.lib.wk_event_create(device, ctypes.byref(self.e1)))

    def close(self):
        self.lib.wk_event_destroy(self.e0)
        self.lib.wk_event_destroy(self.e1)
        self.pipeline.deinit()
        self.ctx.deinit()

    def tensor(self, dtype, host):
        shape = host.shape[:-1] if dtype.startswith("c") else host.shape   # complex: trailing (re, im) axis
        t = self.wk.Tensor.alloc(dtype, self.ctx, self.pipeline, shape)
        self.wk.memory.readFromBuffer(self.pipeline, t, host)
        return t

    def tensor_on_device(self, dtype, shape, seed, full_range=False):
        """A tensor filled on the device by random.uniform (floats in [-1, 1), integers in [-100, 100] or,
        with full_range, over the whole type): the same value ranges as `tensor` of a seeded host array,
        without the host generation and the upload."""
        t = self.wk.Tensor.alloc(dtype, self.ctx, self.pipeline, shape)
        if raw.real_np_dtype(dtype).kind == "f":
            self.wk.random.uniform(self.pipeline, t, seed, -1.0, 1.0)
        elif full_range:
            self.wk.random.uniform(self.pipeline, t, seed)
        else:
            self.wk.random.uniform(self.pipeline, t, seed, -100, 100)
        return t

    def time_ms(self, call, iters, warm_seconds=0.15, repeat=None):
        """ms per call from events on the stream, after keeping the device busy for `warm_seconds`
        (short kernels measured right after an upload see the clocks still ramping).  repeat(n): the
        same call n times from one loop inside the host library, used for the timed launches when given."""
        import time
        t0 = time.perf_counter()
        while True:
            for _ in range(4):
                call()
            self.pipeline.waitAndCleanup()
            if time.perf_counter() - t0 >= warm_seconds:
                break
        check = self.wk._capi.check
        check(self.lib.wk_event_record(self.e0, self.stream))
        if repeat is not None:
            repeat(iters)
        else:
            for _ in range(iters):
                call()
        check(self.lib.wk_event_record(self.e1, self.stream))
        self.pipeline.waitAndCleanup()
        ms = self.ct.c_float()
        check(self.lib.wk_event_elapsed_ms(self.e0, self.e1, self.ct.byref(ms)))
        return ms.value / iters


def time_gemm(ses, dtype, M, N, K, op_a, op_b, alpha, beta, iters=10, device_fill=False, full_range=False, keep_b=False):
    """blas.gemm on tensors created by Tensor.alloc (so with the library's own row pitches).
    device_fill: operands drawn on the device instead of generated on the host and uploaded.
    full_range: integer entries over the whole type instead of [-100, 100] (the integer kernels are exact
    either way, but entries of small magnitude have zero upper digits: the packed 32-bit kernel leaves out
    the digit products of empty planes, and the clock the part holds under the int8 matrix instruction
    depends on how many operand bits toggle).
    keep_b: GemmPackedTensors.keepB(True), i.e. B (the weights of a layer, say) stays packed across the
    calls and only A goes through the pack pass."""
    rd = raw.real_np_dtype(dtype)
    wk = ses.wk
    tail = (2,) if dtype.startswith("c") else ()
    if device_fill:
        A = ses.tensor_on_device(dtype, (K, M) if op_a else (M, K), 1, full_range)
        B = ses.tensor_on_device(dtype, (N, K) if op_b else (K, N), 2, full_range)
        C = ses.tensor_on_device(dtype, (M, N), 3, full_range)
    else:
        A = ses.tensor(dtype, _operand(rd, ((K, M) if op_a else (M, K)) + tail, 1, full_range))
        B = ses.tensor(dtype, _operand(rd, ((N, K) if op_b else (K, N)) + tail, 2, full_range))
        C = ses.tensor(dtype, _operand(rd, (M, N) + tail, 3, full_range))
    # as benchmark/gemm.zig:186-196 does: one GemmPackedTensors for the run, passed to every call
    packed = wk.GemmPackedTensors.init(ses.pipeline, C, K, True)
    if keep_b:
        packed.keepB(True)
    ses.pipeline.waitAndCleanup()
    ms = ses.time_ms(lambda: wk.blas.gemm(ses.pipeline, alpha, A, op_a, B, op_b, beta, C, packed), iters,
                     repeat=lambda n: wk.blas.gemm_repeat(ses.pipeline, alpha, A, op_a, B, op_b, beta, C, packed, n))
    variant = ses.lib.wk_gemm_variant_with_workspace(raw.dtype_id(dtype), op_a, op_b, M, N, K, A.row_pitch, B.row_pitch,
                                                     C.row_pitch, A.buffer, B.buffer, C.buffer,
                                                     packed.workspace_bytes).decode()
    packed.deinit(ses.pipeline)
    for t in (A, B, C):
        t.release(ses.pipeline)
    return ms, variant


def time_axpy(ses, dtype, n, iters=50, device_fill=False, batches=0):
    """n: element count of a 1-D tensor, or a shape tuple (2-D / 3-D tensors have pitched rows).
    batches > 0: that many timed batches of `iters` launches each, returned as a list of ms per call."""
    rd = raw.real_np_dtype(dtype)
    wk = ses.wk
    shape = n if isinstance(n, tuple) else (n,)
    if device_fill:
        x, y = ses.tensor_on_device(dtype, shape, 1), ses.tensor_on_device(dtype, shape, 2)
    else:
        x, y = ses.tensor(dtype, _operand(rd, shape, 1)), ses.tensor(dtype, _operand(rd, shape, 2))
    ses.pipeline.waitAndCleanup()
    alpha = 0.75 if rd.kind == "f" else 3
    once = lambda: wk.blas.axpy(ses.pipeline, x, alpha, y)
    many = lambda count: wk.blas.axpy_repeat(ses.pipeline, x, alpha, y, count)
    if batches:
        ms = [ses.time_ms(once, iters, repeat=many) for _ in range(batches)]
    else:
        ms = ses.time_ms(once, iters, repeat=many)
    x.release(ses.pipeline)
    y.release(ses.pipeline)
    return ms


def cmd_gemm(ses, args):
    print(f"{'dtype':5s} {'n':>6s} {'op':2s} {'ms':>9s} {'TFLOP/s':>9s}  kernel")
    cplx = args.dtype.startswith("c")
    is_float = args.dtype.lstrip("c")[0] == "f"
    alpha, beta = (1.5, 0.5) if is_float else (3, 2)
    if cplx:
        alpha, beta = (alpha, 0.5 if is_float else 1), (beta, 0.25 if is_float else -1)
    ops = 8.0 if cplx else 2.0   # a complex multiply-add counted as four real ones
    shapes = [(n, n, n) for n in args.sizes] if not args.shapes else [tuple(int(v) for v in sh.split("x")) for sh in args.shapes]
    for M, N, K in shapes:
        for op_a, op_b, name in OPS:
            if args.ops and name not in args.ops:
                continue
            ms, variant = time_gemm(ses, args.dtype, M, N, K, op_a, op_b, alpha, beta, device_fill=True, full_range=args.full_range)
            label = str(M) if M == N == K else f"{M}x{N}x{K}"
            print(f"{args.dtype:5s} {label:>6s} {name:2s} {ms:9.4f} {ops * M * N * K / ms / 1e9:9.2f}  {variant}", flush=True)


def cmd_axpy(ses, args):
    print(f"{'dtype':5s} {'n':>10s} {'us':>9s} {'GB/s':>8s}")
    for lg in range(12, 29):
        n = 1 << lg
        ms = time_axpy(ses, args.dtype, n)
        nbytes = 3 * n * raw.elem_size(args.dtype)
        print(f"{args.dtype:5s} {n:10d} {ms * 1e3:9.2f} {nbytes / ms / 1e6:8.0f}", flush=True)
    for shape in ((8192, 8192), (4096, 4096), (2048, 4096), (1000, 1000), (16, 1024, 4096)):
        ms = time_axpy(ses, args.dtype, shape)
        nbytes = 3 * int(np.prod(shape)) * raw.elem_size(args.dtype)
        print(f"{args.dtype:5s} {'x'.join(map(str, shape)):>10s} {ms * 1e3:9.2f} {nbytes / ms / 1e6:8.0f}", flush=True)


# Published MI355X peaks the rates are held against.  32-bit integer products run as ten int8 digit
# products on the matrix cores, so their rate in int8 operations is ten times the 32-bit one.
PEAK = {"f32": (157.3, "TFLOP/s", "mfma", 1.0), "f64": (78.6, "TFLOP/s", "mfma", 1.0), "i32": (5000.0, "TOP/s", "mfma", 10.0)}
HBM_PEAK_GBS = 8000.0


def baseline_gemm_cases():
    """(key, dtype, M, N, K, op_a, op_b, alpha, beta) for every GEMM of the benchmark configurations, in the
    sweep order of benchmark/gemm.zig:240-283 (size outermost, the four op pairs inside).  A key that ends in
    `_full_range` draws its integer entries over the whole type instead of [-100, 100]; one that ends in
    `_b_kept` keeps B packed across the calls (GemmPackedTensors.keepB), so that only A is packed per call."""
    cases = [("1_f32_gemm_512_NN", "f32", 512, 512, 512, 0, 0, 1.0, 0.0)]
    for n in (1024, 2048, 4096, 8192):
        for op_a, op_b, name in OPS:
            cases.append((f"3_f32_gemm_{n}_{name}", "f32", n, n, n, op_a, op_b, 1.5, 0.5))
    for (M, N, K) in ((1000, 1000, 1000), (4097, 4095, 4093)):
        for op_a, op_b, name in OPS:
            cases.append((f"3_f32_gemm_{M}x{N}x{K}_{name}", "f32", M, N, K, op_a, op_b, 1.5, 0.5))
    cases.append(("4_f64_gemm_4096_NN", "f64", 4096, 4096, 4096, 0, 0, 1.0, 1.0))
    cases.append(("4_f64_gemm_8192x256x8192_NN", "f64", 8192, 256, 8192, 0, 0, 1.0, 1.0))
    cases.append(("4_i32_gemm_2048_NN", "i32", 2048, 2048, 2048, 0, 0, 3, -2))
    cases.append(("4_i32_gemm_2048_NN_full_range", "i32", 2048, 2048, 2048, 0, 0, 3, -2))
    cases.append(("4_i32_gemm_2048_NN_b_kept", "i32", 2048, 2048, 2048, 0, 0, 3, -2))
    return cases


def run_baseline_configs(ses, log=None, device_fill=True):
    """Every GEMM and AXPY benchmark configuration, each with its own roofline figures.  Returns a dict
    key -> {ms, value, unit, kernel, roofline}."""
    out = {}
    for key, dtype, M, N, K, op_a, op_b, alpha, beta in baseline_gemm_cases():
        ms, variant = time_gemm(ses, dtype, M, N, K, op_a, op_b, alpha, beta, device_fill=device_fill,
                                full_range=key.endswith("_full_range"), keep_b=key.endswith("_b_kept"))
        peak, unit, bound, scale = PEAK[dtype]
        issued = None
        if dtype == "i32":
            # digit products the packed kernel issues per element product: all ten pairs (i, j), i + j <= 3, when
            # the entries fill the type; the single pair (0, 0) when every entry is one balanced digit ([-128, 127])
            issued = 10 if key.endswith("_full_range") else 1
            scale = float(issued)
        rate = 2.0 * M * N * K / ms / 1e9
        out[key] = {"ms": ms, "value": rate, "unit": unit, "kernel": variant,
                    "roofline": {"bound": bound, "achieved": rate * scale, "peak": peak, "unit": unit,
                                 "frac": rate * scale / peak}}
        if issued is not None:
            out[key]["roofline"]["digit_products_issued"] = issued
            out[key]["roofline"]["note"] = ("achieved = 32-bit operations x int8 digit products issued per element product, "
                                            "against the int8 matrix peak; the pack pass is inside the time")
        if raw.real_np_dtype(dtype).kind != "f":
            out[key]["entries"] = "uniform over the whole type" if key.endswith("_full_range") else "uniform in [-100, 100]"
        if log:
            log(f"{key}: {ms:.4f} ms -> {rate:.1f} {unit} = {100 * rate * scale / peak:.1f} % of peak [{variant}]")
    for dt in ("f32", "f64"):
        for lg in (20, 24, 28):
            nbytes = 3.0 * (1 << lg) * raw.elem_size(dt)
            spread = None
            if lg >= 28:
                # which side of a percent a single batch lands on is the box's: seven batches, the median counts
                times = sorted(time_axpy(ses, dt, 1 << lg, iters=20, device_fill=device_fill, batches=7))
                ms = times[len(times) // 2]
                spread = {"batches": len(times), "launches_per_batch": 20, "median": nbytes / ms / 1e6,
                          "min": nbytes / times[-1] / 1e6, "max": nbytes / times[0] / 1e6, "unit": "GB/s"}
            else:
                ms = time_axpy(ses, dt, 1 << lg, device_fill=device_fill)
            rate = nbytes / ms / 1e6
            key = f"2_axpy_{dt}_2p{lg}"
            out[key] = {"ms": ms, "value": rate, "unit": "GB/s", "kernel": "axpy_stream", "bytes_per_launch": nbytes,
                        "roofline": {"bound": "hbm", "achieved": rate, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                     "frac": rate / HBM_PEAK_GBS}}
            if spread:
                out[key]["over_batches"] = spread
            if log:
                log(f"{key}: {ms * 1e3:.1f} us -> {rate:.0f} GB/s = {100 * rate / HBM_PEAK_GBS:.1f} % of HBM peak")
    return out


def off_benchmark_gemm_cases():
    """(dtype, M, N, K, op_a, op_b) of products that are not among the benchmark configurations: squares with
    sides between the powers of two, where the tiles do not fill whole rounds of the device and the choice of a
    kernel is what counts, and small batches against a large matrix (Linear.forward at batch sizes up to 32)."""
    cases = [("f32", n, n, n, 0, 0) for n in (1100, 1536, 2300, 2500, 3200, 4300, 6000)]
    cases += [("f32", 2300, 2300, 2300, 1, 0), ("f32", 2300, 2300, 2300, 0, 1)]
    cases += [("f64", n, n, n, 0, 0) for n in (1100, 1536, 2300, 3456, 4300)]
    cases += [("f32", 32, 8192, 8192, 0, 1), ("f32", 16, 8192, 8192, 0, 1), ("f32", 8, 4096, 4096, 0, 1), ("f32", 1, 8192, 8192, 0, 1),
              ("f64", 32, 8192, 8192, 0, 1), ("f64", 8, 4096, 4096, 0, 1)]
    return cases


def run_off_benchmark_sizes(ses, log=None):
    """The products of off_benchmark_gemm_cases, timed like the benchmark configurations.  Returns a dict
    key -> {ms, value, unit, kernel, frac}; products of at most 32 rows, which wait for memory, also carry the
    rate at which their large operand is read (`operand_GBs`)."""
    out = {}
    names = {(a, b): name for a, b, name in OPS}
    for dtype, M, N, K, op_a, op_b in off_benchmark_gemm_cases():
        ms, variant = time_gemm(ses, dtype, M, N, K, op_a, op_b, 1.5, 0.5, device_fill=True)
        peak, unit, _, _ = PEAK[dtype]
        rate = 2.0 * M * N * K / ms / 1e9
        shape = str(M) if M == N == K else f"{M}x{N}x{K}"
        key = f"{dtype}_gemm_{shape}_{names[(op_a, op_b)]}"
        out[key] = {"ms": ms, "value": rate, "unit": unit, "kernel": variant, "frac": rate / peak}
        note = f"{100 * rate / peak:.1f} % of peak"
        if min(M, N) <= 32:
            gbs = max(M, N) * K * raw.elem_size(dtype) / ms / 1e6
            out[key]["operand_GBs"] = gbs
            out[key]["operand_frac_of_hbm_peak"] = gbs / HBM_PEAK_GBS
            note = f"large operand read at {gbs:.0f} GB/s = {100 * gbs / HBM_PEAK_GBS:.1f} % of HBM peak"
        if log:
            log(f"{key}: {ms:.4f} ms -> {rate:.1f} {unit}, {note} [{variant}]")
    return out


def cmd_configs(ses, args):
    rows = run_baseline_configs(ses, device_fill=False)
    print(f"{'config':38s} {'ms':>9s} {'rate':>9s} unit     % peak  kernel")
    for name, r in rows.items():
        print(f"{name:38s} {r['ms']:9.4f} {r['value']:9.2f} {r['unit']:8s} {100 * r['roofline']['frac']:6.1f}  {r['kernel']}")


NARROW_SHAPES = [(1, 8192, 8192), (4, 8192, 8192), (8, 4096, 4096), (16, 8192, 8192), (32, 8192, 8192), (24, 4096, 16384),
                 (32, 2048, 2048), (16, 16384, 1024), (8192, 32, 8192), (4096, 8, 4096), (8192, 4, 8192)]


def cmd_narrow(ses, args):
    """Products with at most 32 rows or columns of C against a large other operand (small batches through a
    weight matrix): the automatic choice beside the same call with the skinny kernel switched off (the thin
    kernel up to four rows or columns, the 64 x 64 tile kernels beyond), and the rate at which the large
    operand is read."""
    did = raw.dtype_id(args.dtype)
    sz = raw.elem_size(args.dtype)
    print(f"{'dtype':5s} {'shape':>16s} {'op':2s} {'us':>8s} {'TB/s':>6s}  {'kernel':8s} | {'us':>8s}  kernel without the skinny kernel")
    for M, N, K in NARROW_SHAPES:
        for op_a, op_b, name in OPS:
            if args.ops and name not in args.ops:
                continue
            rows = []
            for skinny in (1, 0):
                raw.check(ses.lib.wk_test_option(b"skinny", skinny), "wk_test_option")
                try:
                    rows.append(time_gemm(ses, args.dtype, M, N, K, op_a, op_b, 1.5, 0.5, iters=20, device_fill=True))
                finally:
                    ses.lib.wk_test_option(b"skinny", 1)
            (ms, kernel), (ms0, kernel0) = rows
            print(f"{args.dtype:5s} {f'{M}x{N}x{K}':>16s} {name:2s} {ms * 1e3:8.1f} {max(M, N) * K * sz / ms / 1e9:6.2f}  {kernel:8s} | "
                  f"{ms0 * 1e3:8.1f}  {kernel0}", flush=True)


REGRET_SHAPES = [(512, 2048), (1000, 3000), (1536, 1536), (2048, 1024), (3000, 1000), (1280, 5000), (4096, 2048), (6000, 1500), (2500, 2500),
                 (3072, 5120), (700, 9000), (5000, 5000), (1792, 3584), (1100, 1100), (8192, 1024), (3333, 2222)]
REGRET_VARIANTS = {"f32": ["256x128d", "128x128d", "64x64d", "128x128d2", "64x64d2", "32x32s4", "64x64z", "256x128k", "128x128k", "64x64k"],
                   "f64": ["128x128d", "64x64d", "32x32s4", "64x64z", "128x128k", "64x64k", "64x64s2"]}


def cmd_regret(ses, args):
    """How far the automatic choice of a kernel is behind the best forced one: M x N of REGRET_SHAPES x the given
    values of k x N,N / T,N, six launches per point.  Prints the points above the threshold and the mean."""
    def timed(M, N, K, op_a, op_b, variant):
        ses.lib.wk_gemm_force_variant(f"mfma_{args.dtype}_{variant}".encode() if variant else b"auto")
        try:
            return time_gemm(ses, args.dtype, M, N, K, op_a, op_b, 1.5, 0.5, iters=6, device_fill=True)
        except Exception:   # a variant that does not take the shape
            return float("inf"), "-"
        finally:
            ses.lib.wk_gemm_force_variant(b"auto")
    total, points, above = 0.0, 0, 0
    for M, N in REGRET_SHAPES:
        for K in args.ks:
            for op_a, op_b, name in OPS:
                if name not in ("NN", "TN"):
                    continue
                auto_ms, auto_name = timed(M, N, K, op_a, op_b, None)
                best_ms, best_name = auto_ms, "auto"
                for v in REGRET_VARIANTS[args.dtype]:
                    if M * N * K > 4e10 and v in ("32x32s4", "64x64z", "64x64s2"):   # (minutes per launch, never the best there)
                        continue
                    ms, _ = timed(M, N, K, op_a, op_b, v)
                    if ms < best_ms:
                        best_ms, best_name = ms, v
                behind = auto_ms / best_ms - 1.0
                total += behind
                points += 1
                if behind > args.threshold:
                    above += 1
                    print(f"{args.dtype} {M}x{N}x{K} {name}: automatic {auto_name} {auto_ms * 1e3:.1f} us, best {best_name} {best_ms * 1e3:.1f} us, "
                          f"{100 * behind:.1f} % behind", flush=True)
    print(f"{args.dtype}: {points} points, {100 * total / points:.2f} % behind on average, {above} above {100 * args.threshold:.0f} %", flush=True)


def cmd_tensor(ses, args):
    """Streaming rates of the tensor support operations (algorithmic bytes: one read and one write of
    every element, one write for random.uniform)."""
    wk = ses.wk
    print(f"{'operation':44s} {'us':>9s} {'GB/s':>8s}")
    for dtype, shape, d0, d1 in (("f32", (8192, 8192), 0, 1), ("f64", (8192, 8192), 0, 1), ("cf64", (4096, 4096), 0, 1),
                                 ("u8", (16384, 16384), 0, 1), ("f32", (64, 1024, 1024), 0, 1), ("f32", (64, 1024, 1024), 1, 2),
                                 ("f32", (1024, 64, 1024), 0, 2)):
        x = wk.Tensor.alloc(dtype, ses.ctx, ses.pipeline, shape)
        rshape = list(shape)
        rshape[d0], rshape[d1] = rshape[d1], rshape[d0]
        r = wk.Tensor.alloc(dtype, ses.ctx, ses.pipeline, rshape)
        wk.random.uniform(ses.pipeline, x, 1)
        ms = ses.time_ms(lambda: wk.transpose(ses.pipeline, r, x, d0, d1), 20)
        nbytes = 2.0 * np.prod(shape) * raw.elem_size(dtype)
        print(f"{'transpose ' + dtype + ' ' + 'x'.join(map(str, shape)) + f' dims {d0},{d1}':44s} {ms * 1e3:9.1f} {nbytes / ms / 1e6:8.0f}",
              flush=True)
        x.release(ses.pipeline)
        r.release(ses.pipeline)
    x = wk.Tensor.alloc("f32", ses.ctx, ses.pipeline, (8192, 8192))
    y = wk.Tensor.alloc("f32", ses.ctx, ses.pipeline, (8192, 8192))
    z = wk.Tensor.alloc("cf32", ses.ctx, ses.pipeline, (8192, 8192))
    n = 8192.0 * 8192
    for name, call, nbytes in (
            ("memory.copy f32 8192x8192", lambda: wk.memory.copy(ses.pipeline, x, y), 8 * n),
            ("random.uniform f32 8192x8192", lambda: wk.random.uniform(ses.pipeline, x, 7), 4 * n),
            ("random.uniform f32 8192x8192 in [-1, 1]", lambda: wk.random.uniform(ses.pipeline, x, 7, -1.0, 1.0), 4 * n),
            ("random.uniform cf32 8192x8192", lambda: wk.random.uniform(ses.pipeline, z, 7), 8 * n),
            ("toComplex f32 -> cf32 8192x8192", lambda: wk.convertions.toComplex(ses.pipeline, x, z, wk.Space.real), 8 * n),
            ("toReal cf32 -> f32 8192x8192", lambda: wk.convertions.toReal(ses.pipeline, z, x, wk.Space.imag), 8 * n)):
        ms = ses.time_ms(call, 20)
        print(f"{name:44s} {ms * 1e3:9.1f} {nbytes / ms / 1e6:8.0f}", flush=True)
    for t in (x, y, z):
        t.release(ses.pipeline)


def mlp_flops(sizes, batch):
    """Multiply-adds of the GEMMs of one training step, as flops: forward and weight gradients over
    every layer, input sensitivities over every layer but the first."""
    pairs = list(zip(sizes[:-1], sizes[1:]))
    fwd = sum(2.0 * batch * i * o for i, o in pairs)
    return 2 * fwd + sum(2.0 * batch * i * o for i, o in pairs[1:])


def time_mlp_step(dtype="f32", sizes=(1024, 4096, 4096, 1024), batch=2048, optimizer="adam", lr=1e-3, steps=20, warmup=3,
                  seed=None):
    """One training step of benchmark configuration 5 through the reference-shaped API: Sequential of
    Linear layers (tanh hidden, sigmoid output), loss.mse with derivative, backward, optimizer step.
    Returns ms per step from events on the pipeline's stream and from the wall clock."""
    import ctypes
    import time

    import wekua_amd as wk
    from wekua_amd import nn

    seed = synth.config_seed(5, 0) if seed is None else seed
    rd = raw.real_np_dtype(dtype)
    ctx = wk.Context.initFromDeviceType(wk.DeviceType.all)
    pipeline = wk.Pipeline.init(ctx.command_queues[0])
    seq = nn.Sequential.init(dtype)
    n_layers = len(sizes) - 1
    for i in range(n_layers):
        act = nn.Sigmoid.init() if i == n_layers - 1 else nn.Tanh.init()
        seq.append(nn.Linear.init(dtype, ctx, pipeline, sizes[i], sizes[i + 1], act, seed=seed + i))
    x = wk.Tensor.alloc(dtype, ctx, pipeline, (batch, sizes[0]))
    y = wk.Tensor.alloc(dtype, ctx, pipeline, (batch, sizes[-1]))
    wk.memory.readFromBuffer(pipeline, x, synth.normal(synth.config_seed(5, 8), (batch, sizes[0]), rd))
    wk.memory.readFromBuffer(pipeline, y, synth.uniform(synth.config_seed(5, 9), (batch, sizes[-1]), rd, 0.0, 1.0))
    cache = nn.Cache.init(ctx, pipeline, batch, [seq])
    lc = cache.getLayerCache(0)
    opt = nn.optimizers.Adam.init(dtype, lr) if optimizer == "adam" else nn.optimizers.GD.init(dtype, lr)

    def step():
        out = seq.forward(pipeline, x, lc)
        nn.loss.mse(True, pipeline, out, y, cache, None)
        seq.backward(pipeline, lc, x, None)
        opt.step(pipeline, cache)

    for _ in range(warmup):
        step()
    pipeline.waitAndCleanup()
    lib = wk._capi.load()
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
    loss = np.zeros(1, dtype=rd)
    nn.loss.mse(False, pipeline, seq.forward(pipeline, x, lc), y, cache, loss)
    lib.wk_event_destroy(e0)
    lib.wk_event_destroy(e1)
    opt.deinit(pipeline)
    cache.deinit(pipeline)
    seq.deinit(pipeline)
    x.release(pipeline)
    y.release(pipeline)
    pipeline.deinit()
    ctx.deinit()
    flops = mlp_flops(sizes, batch)
    return {"stream_ms": ms.value / steps, "wall_ms": wall_ms, "flops": flops, "tflops": flops / (ms.value / steps) / 1e9,
            "loss_after": float(loss[0])}


def cmd_probe(ses, args):
    """What a launch costs before any product is computed: an empty kernel and a kernel that only stores an
    f32 tile per work-group, on the grids, work-group sizes and LDS claims of the small one-round GEMM launches;
    per-call time on the stream (back-to-back launches, like the GEMM rows of this benchmark)."""
    import ctypes
    wk = ses.wk
    dev = wk._lib().wkz_context_device(ses.ctx._h)
    buf = ctypes.c_void_p()
    nbytes = 64 << 20
    wk._capi.check(ses.lib.wk_malloc(dev, nbytes, ctypes.byref(buf)))
    print(f"{'probe':12s} {'work-groups':>11s} {'threads':>7s} {'LDS KiB':>7s} {'us':>7s}")
    for wgs, threads, lds_kib in ((256, 256, 0), (256, 256, 48), (256, 512, 96), (256, 1024, 96), (64, 256, 48), (1024, 256, 48),
                                  (2048, 256, 72)):
        for kind, name in ((0, "empty"), (1, "store-only")):
            check = wk._capi.check

            def batch(iters):
                check(ses.lib.wk_event_record(ses.e0, ses.stream))
                for _ in range(iters):
                    check(ses.lib.wk_probe_launch(ses.stream, kind, wgs, threads, lds_kib << 10, buf, nbytes))
                check(ses.lib.wk_event_record(ses.e1, ses.stream))
                check(ses.lib.wk_stream_sync(ses.stream))     # these launches do not go through the pipeline
                t = ctypes.c_float()
                check(ses.lib.wk_event_elapsed_ms(ses.e0, ses.e1, ctypes.byref(t)))
                return t.value / iters
            batch(200)
            ms = min(batch(50) for _ in range(3))
            print(f"{name:12s} {wgs:11d} {threads:7d} {lds_kib:7d} {ms * 1e3:7.2f}", flush=True)
    wk._capi.check(ses.lib.wk_free(dev, buf))


def cmd_mlp(args):
    r = time_mlp_step(args.dtype, tuple(args.sizes), args.batch, args.optimizer, args.lr, args.steps, args.warmup)
    print(f"mlp {'-'.join(map(str, args.sizes))} {args.dtype} batch {args.batch} {args.optimizer}: "
          f"{r['stream_ms']:.3f} ms/step on the stream, {r['wall_ms']:.3f} ms/step wall, "
          f"{r['tflops']:.1f} TFLOP/s over {r['flops'] / 1e9:.1f} GFLOP of GEMM work, "
          f"mse after {args.steps + args.warmup} steps {r['loss_after']:.5f}")


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m wekua_amd.benchmark")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("gemm")
    g.add_argument("--dtype", default="f32")
    g.add_argument("--sizes", type=int, nargs="+", default=[4 << i for i in range(4, 12)])
    g.add_argument("--variant", default="auto")
    g.add_argument("--shapes", nargs="+", default=None, help="MxNxK ... instead of the square --sizes")
    g.add_argument("--ops", nargs="+", default=None, choices=["NN", "NT", "TN", "TT"], help="only these operand layouts")
    g.add_argument("--full-range", action="store_true", help="integer entries over the whole type instead of [-100, 100]")
    a = sub.add_parser("axpy")
    a.add_argument("--dtype", default="f32")
    sub.add_parser("tensor")
    r = sub.add_parser("regret")
    r.add_argument("--dtype", default="f32", choices=["f32", "f64"])
    r.add_argument("--ks", type=int, nargs="+", default=[384, 1024, 2500, 6000])
    r.add_argument("--threshold", type=float, default=0.04)
    n = sub.add_parser("narrow")
    n.add_argument("--dtype", default="f32", choices=["f32", "f64"])
    n.add_argument("--ops", nargs="+", default=None, choices=["NN", "NT", "TN", "TT"], help="only these operand layouts")
    sub.add_parser("probe")
    c = sub.add_parser("configs")
    c.add_argument("--variant", default="auto")
    m = sub.add_parser("mlp")
    m.add_argument("--dtype", default="f32")
    m.add_argument("--sizes", type=int, nargs="+", default=[1024, 4096, 4096, 1024])
    m.add_argument("--batch", type=int, default=2048)
    m.add_argument("--optimizer", choices=["adam", "gd"], default="adam")
    m.add_argument("--lr", type=float, default=1e-3)
    m.add_argument("--steps", type=int, default=20)
    m.add_argument("--warmup", type=int, default=3)
    args = ap.parse_args(argv)
    if args.cmd == "mlp":
        cmd_mlp(args)
        return 0
    ses = Session()
    try:
        if getattr(args, "variant", "auto") != "auto":
            raw.check(ses.lib.wk_gemm_force_variant(args.variant.encode()), "wk_gemm_force_variant")
        {"gemm": cmd_gemm, "axpy": cmd_axpy, "configs": cmd_configs, "tensor": cmd_tensor, "probe": cmd_probe, "narrow": cmd_narrow, "regret": cmd_regret}[args.cmd](ses, args)
    finally:
        ses.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
