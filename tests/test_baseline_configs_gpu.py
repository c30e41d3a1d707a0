"""GPU: the benchmark configurations at their real sizes.

Every shape, 8192^3 included, is compared entry by entry with the oracle's reference-order product
(threaded, it finishes 8192^3 in seconds), both through the mirrored API (the library's own pitches:
what the benchmark figures are measured on) and through the C ABI with unpadded leading dimensions.
A float64 second opinion that does not go through the C oracle is taken on one layout per shape:
  * a lattice of entries -- one in every 32x32 block of C, walking through every position of a block,
    plus the last row and column -- against float64 dot products (tolerance 1e-5*sqrt(K) /
    1e-12*sqrt(K) relative to sum|a||b|, as stated for the task);
  * every entry, in aggregate: C @ 1 must equal alpha * A (B 1) + beta * C0 1 (linearity), an
    O(n^2) identity evaluated in float64.
int32 is compared bit for bit: for |entries| <= 2^20 and K = 2048 every partial sum stays
below 2^53, so a float64 product is exact and is then reduced mod 2^32.
"""
import numpy as np
import pytest

import oracle
from helpers import (F32_TOL, F64_TOL, assert_every_entry, assert_gemm_close, gemm_bound_fast,
                     lattice_errors)
from wekua_amd import synth

pytestmark = pytest.mark.gpu
OPS = [(0, 0), (0, 1), (1, 0), (1, 1)]


def run(dev, dtype, alpha, a, op_a, b, op_b, beta, c):
    M, N = c.shape
    K = a.shape[0] if op_a else a.shape[1]
    dA, dB, dC = dev.upload(a), dev.upload(b), dev.upload(c)
    dev.gemm(dtype, op_a, op_b, M, N, K, alpha, dA, a.shape[1], dB, b.shape[1], beta, dC, N)
    out = dC.download(c.dtype, c.shape)
    for d in (dA, dB, dC):
        d.free()
    return out


def operands(rd, M, N, K, op_a, op_b, cfg):
    a = synth.uniform(synth.config_seed(cfg, 0), (K, M) if op_a else (M, K), rd)
    b = synth.uniform(synth.config_seed(cfg, 1), (N, K) if op_b else (K, N), rd)
    c = synth.uniform(synth.config_seed(cfg, 2), (M, N), rd)
    return a, b, c


def check_by_properties(dtype, got, alpha, a, op_a, b, op_b, beta, c, K):
    """A float64 second opinion that is independent of the C oracle: a lattice of entries (one in every 32x32
    block of C, walking through every position of such a block, plus the whole last row and column) against
    float64 dot products, and the row / column sums of all entries (linearity)."""
    tol = (F32_TOL if dtype == "f32" else F64_TOL) * np.sqrt(K)
    assert np.isfinite(got).all()
    A = a.T if op_a else a
    B = b.T if op_b else b
    al = 1.0 if alpha is None else float(alpha)
    be = 0.0 if beta is None else float(beta)
    M, N = got.shape
    ii, jj, err = lattice_errors(dtype, got, alpha, a, op_a, b, op_b, beta, c, K)
    worst = int(err.argmax())
    assert err[worst] <= 1.0, f"lattice entry ({ii[worst]}, {jj[worst]}): {err[worst]:.3g} x tolerance"
    # linearity over all entries: row sums
    ones = np.ones(N, dtype=np.float64)
    rhs = al * (A.astype(np.float64) @ (B.astype(np.float64) @ ones)) + be * (c.astype(np.float64) @ ones)
    rb = abs(al) * (np.abs(A).astype(np.float64) @ (np.abs(B).astype(np.float64) @ ones)) + abs(be) * (np.abs(c).astype(np.float64) @ ones)
    lhs = got.astype(np.float64) @ ones
    rerr = np.abs(lhs - rhs) / rb
    assert rerr.max() <= tol, f"row sums: {rerr.max():.3e} > {tol:.3e}"
    # and column sums (catches a transposed block that row sums of a symmetric layout would not)
    onesM = np.ones(M, dtype=np.float64)
    rhs = al * ((onesM @ A.astype(np.float64)) @ B.astype(np.float64)) + be * (onesM @ c.astype(np.float64))
    cb = abs(al) * ((onesM @ np.abs(A).astype(np.float64)) @ np.abs(B).astype(np.float64)) + abs(be) * (onesM @ np.abs(c).astype(np.float64))
    cerr = np.abs(onesM @ got.astype(np.float64) - rhs) / cb
    assert cerr.max() <= tol, f"column sums: {cerr.max():.3e} > {tol:.3e}"


@pytest.fixture(scope="module")
def api():
    """One context + pipeline of the mirrored API: the path bench.py times (the library's own row pitches)."""
    import wekua_amd as wk
    context = wk.Context.initFromDeviceType(wk.DeviceType.all)
    pipeline = wk.Pipeline.init(context.command_queues[0])
    yield wk, context, pipeline
    pipeline.deinit()
    context.deinit()


def run_tensors(api, dtype, alpha, a, op_a, b, op_b, beta, c, expect_variant=None):
    """blas.gemm on Tensor operands (padded, possibly skewed pitches: what the headline figures are measured
    on).  Returns the product and the name of the kernel variant the library chose."""
    from wekua_amd import raw
    wk, context, pipeline = api
    M, N = c.shape
    K = a.shape[0] if op_a else a.shape[1]
    tensors = []
    for host in (a, b, c):
        t = wk.Tensor.alloc(dtype, context, pipeline, host.shape)
        wk.memory.readFromBuffer(pipeline, t, host)
        tensors.append(t)
    A, B, C = tensors
    name = wk._capi.load().wk_gemm_variant(raw.dtype_id(dtype), op_a, op_b, M, N, K, A.row_pitch, B.row_pitch,
                                               C.row_pitch, A.buffer, B.buffer, C.buffer).decode()
    wk.blas.gemm(pipeline, alpha, A, op_a, B, op_b, beta, C, None)
    got = np.empty_like(c)
    wk.memory.writeToBuffer(pipeline, C, got)
    pipeline.waitAndCleanup()
    for t in tensors:
        t.release(pipeline)
    if expect_variant is not None:
        assert expect_variant in name, f"expected a {expect_variant} kernel, the library chose {name}"
    return got, name


def check_whole_product(dtype, got, alpha, a, op_a, b, op_b, beta, c, K, what):
    """Every entry against the oracle's reference-order product (the CPU device's packed path)."""
    vw = 8 if dtype == "f32" else 4
    want = oracle.gemm(dtype, alpha, a, op_a, b, op_b, beta, c, vector_width=vw, packed=True, threads=0)
    bound = gemm_bound_fast(dtype, alpha, a, op_a, b, op_b, beta, c)
    assert_every_entry(dtype, got, want, bound, K, what=what)


def test_config1_f32_512(dev):
    """f32 C = 1.0*A*B + 0.0*C at 512^3 (C initially zero), also the reference CPU path's own case."""
    a, b, _ = operands(np.float32, 512, 512, 512, 0, 0, 1)
    c = np.zeros((512, 512), np.float32)
    got = run(dev, "f32", 1.0, a, 0, b, 0, 0.0, c)
    want = oracle.gemm("f32", 1.0, a, 0, b, 0, 0.0, c, vector_width=8, packed=True)   # the CPU device's own path
    assert_gemm_close("f32", got, want, 1.0, a, 0, b, 0, 0.0, c, 512, what="config 1")
    exact = oracle.semantic_gemm("f32", 1.0, a, 0, b, 0, 0.0, c)     # long-double accumulation
    assert_gemm_close("f32", got, exact, 1.0, a, 0, b, 0, 0.0, c, 512, what="config 1 vs exact")


@pytest.mark.parametrize("n", [1024, 2048])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_config3_f32_square_vs_oracle(dev, api, n, op_a, op_b):
    a, b, c = operands(np.float32, n, n, n, op_a, op_b, 3)
    got = run(dev, "f32", 1.5, a, op_a, b, op_b, 0.5, c)
    want = oracle.gemm("f32", 1.5, a, op_a, b, op_b, 0.5, c, vector_width=8, packed=True)
    assert_gemm_close("f32", got, want, 1.5, a, op_a, b, op_b, 0.5, c, n, what=f"config 3 n={n}")
    got, name = run_tensors(api, "f32", 1.5, a, op_a, b, op_b, 0.5, c)
    assert_gemm_close("f32", got, want, 1.5, a, op_a, b, op_b, 0.5, c, n, what=f"config 3 n={n} tensors ({name})")


@pytest.mark.parametrize("n", [4096, 8192])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_config3_f32_square_large_every_entry(dev, api, n, op_a, op_b):
    """4096^3 and 8192^3, all four layouts, every entry of C against the oracle: once through the mirrored API
    (the kernel and the pitches of the headline figure) and once through the C ABI with unpadded leading
    dimensions."""
    print(f"f32 {n}^3 op=({op_a},{op_b})", flush=True)
    a, b, c = operands(np.float32, n, n, n, op_a, op_b, 3)
    want = oracle.gemm("f32", 1.5, a, op_a, b, op_b, 0.5, c, vector_width=8, packed=True, threads=0)
    bound = gemm_bound_fast("f32", 1.5, a, op_a, b, op_b, 0.5, c)
    got, name = run_tensors(api, "f32", 1.5, a, op_a, b, op_b, 0.5, c, expect_variant="256x128d")
    assert_every_entry("f32", got, want, bound, n, what=f"config 3 n={n} tensors ({name})")
    if (op_a, op_b) == (0, 0):
        check_by_properties("f32", got, 1.5, a, op_a, b, op_b, 0.5, c, n)      # float64, independent of the oracle
    got = run(dev, "f32", 1.5, a, op_a, b, op_b, 0.5, c)
    assert_every_entry("f32", got, want, bound, n, what=f"config 3 n={n} C ABI")


@pytest.mark.parametrize("op_a,op_b", OPS)
def test_config3_f32_ragged_1000(dev, api, op_a, op_b):
    a, b, c = operands(np.float32, 1000, 1000, 1000, op_a, op_b, 3)
    got = run(dev, "f32", 1.5, a, op_a, b, op_b, 0.5, c)
    want = oracle.gemm("f32", 1.5, a, op_a, b, op_b, 0.5, c, vector_width=8, packed=True)
    assert_gemm_close("f32", got, want, 1.5, a, op_a, b, op_b, 0.5, c, 1000, what="config 3 1000^3")
    got, name = run_tensors(api, "f32", 1.5, a, op_a, b, op_b, 0.5, c)
    assert_gemm_close("f32", got, want, 1.5, a, op_a, b, op_b, 0.5, c, 1000, what=f"config 3 1000^3 tensors ({name})")


@pytest.mark.parametrize("op_a,op_b", OPS)
def test_config3_f32_ragged_4097x4095x4093_every_entry(dev, api, op_a, op_b):
    """The ragged configuration: every entry, through the mirrored API (body of whole tiles on the direct-to-LDS
    kernel + the strip of one row as a product of its own) and through the C ABI with lda = K etc. (rows that
    do not start on 16-byte boundaries)."""
    M, N, K = 4097, 4095, 4093
    print(f"f32 {M}x{N}x{K} op=({op_a},{op_b})", flush=True)
    a, b, c = operands(np.float32, M, N, K, op_a, op_b, 3)
    want = oracle.gemm("f32", 1.5, a, op_a, b, op_b, 0.5, c, vector_width=8, packed=True, threads=0)
    bound = gemm_bound_fast("f32", 1.5, a, op_a, b, op_b, 0.5, c)
    got, name = run_tensors(api, "f32", 1.5, a, op_a, b, op_b, 0.5, c)
    assert_every_entry("f32", got, want, bound, K, what=f"4097x4095x4093 tensors ({name})")
    if (op_a, op_b) == (1, 0):
        check_by_properties("f32", got, 1.5, a, op_a, b, op_b, 0.5, c, K)
    got = run(dev, "f32", 1.5, a, op_a, b, op_b, 0.5, c)
    assert_every_entry("f32", got, want, bound, K, what="4097x4095x4093 C ABI")


@pytest.mark.parametrize("op_a,op_b", OPS)
def test_config4_f64_4096_every_entry(dev, api, op_a, op_b):
    print(f"f64 4096^3 op=({op_a},{op_b})", flush=True)
    a, b, c = operands(np.float64, 4096, 4096, 4096, op_a, op_b, 4)
    got, name = run_tensors(api, "f64", 1.0, a, op_a, b, op_b, 1.0, c, expect_variant="128x128d")
    check_whole_product("f64", got, 1.0, a, op_a, b, op_b, 1.0, c, 4096, f"f64 4096^3 tensors ({name})")
    if (op_a, op_b) == (0, 0):
        check_by_properties("f64", got, 1.0, a, 0, b, 0, 1.0, c, 4096)
        got = run(dev, "f64", 1.0, a, 0, b, 0, 1.0, c)
        check_whole_product("f64", got, 1.0, a, 0, b, 0, 1.0, c, 4096, "f64 4096^3 C ABI")


def test_config4_f64_tall_skinny_every_entry(dev, api):
    M, N, K = 8192, 256, 8192
    a, b, c = operands(np.float64, M, N, K, 0, 0, 4)
    got, name = run_tensors(api, "f64", 1.0, a, 0, b, 0, 1.0, c)
    check_whole_product("f64", got, 1.0, a, 0, b, 0, 1.0, c, K, f"f64 8192x256x8192 tensors ({name})")
    got = run(dev, "f64", 1.0, a, 0, b, 0, 1.0, c)
    check_whole_product("f64", got, 1.0, a, 0, b, 0, 1.0, c, K, "f64 8192x256x8192 C ABI")
    check_by_properties("f64", got, 1.0, a, 0, b, 0, 1.0, c, K)
    # small enough for a full float64 reference as well (numpy's own BLAS, a third opinion)
    ref = a @ b + c
    bound = np.abs(a) @ np.abs(b) + np.abs(c)
    assert (np.abs(got - ref) / bound).max() <= F64_TOL * np.sqrt(K)


def _exact_int32(alpha, a, b, beta, c):
    prod = a.astype(np.float64) @ b.astype(np.float64)          # exact: every partial sum < 2^53
    assert np.abs(prod).max() < 2.0 ** 53
    p = prod.astype(np.int64)
    al = 1 if alpha is None else alpha
    out = p * al + (0 if beta is None else beta) * c.astype(np.int64)
    if alpha is None and beta is None:
        out = p
    return (out & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


@pytest.mark.parametrize("alpha,beta", [(None, None), (3, -2)])
def test_config4_int32_2048_bit_exact(dev, alpha, beta):
    n = 2048
    a = synth.integers(synth.config_seed(4, 3), (n, n), np.int32, -100, 100)
    b = synth.integers(synth.config_seed(4, 4), (n, n), np.int32, -100, 100)
    c = synth.integers(synth.config_seed(4, 5), (n, n), np.int32, -100, 100)
    got = run(dev, "i32", alpha, a, 0, b, 0, beta, c)
    assert np.array_equal(got, _exact_int32(alpha, a, b, beta, c))


def test_config4_int32_overflow_forcing(dev):
    """Entries up to 2^20 with K = 2048: products reach 2^40 and sums wrap many times."""
    M, N, K = 512, 384, 2048
    a = synth.integers(11, (M, K), np.int32, -2 ** 20, 2 ** 20)
    b = synth.integers(12, (K, N), np.int32, -2 ** 20, 2 ** 20)
    c = synth.integers(13, (M, N), np.int32, -2 ** 31, 2 ** 31 - 1)
    want = _exact_int32(65537, a, b, -3, c)
    assert (np.abs(a.astype(np.float64) @ b.astype(np.float64)) > 2.0 ** 31).any()   # it really overflows
    got = run(dev, "i32", 65537, a, 0, b, 0, -3, c)
    assert np.array_equal(got, want)
    # the C restatement of the reference's kernels wraps identically
    assert np.array_equal(oracle.gemm("i32", 65537, a, 0, b, 0, -3, c), want)


@pytest.mark.parametrize("shape", [(4096, 4096, 2048), (2048, 2048, 2048), (2125, 1541, 1090)])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_config4_int32_large_with_packed_tensors(op_a, op_b, shape):
    """The int32 product the way benchmark/gemm.zig drives it: through blas.gemm with a
    GemmPackedTensors, at sizes where the library takes its pack pass + packed kernel: configuration 4's
    own 2048^3, a larger one, and a ragged one whose 35 k-slabs are padded to an even count."""
    import wekua_amd as wk
    from wekua_amd import raw
    M, N, K = shape
    a = synth.integers(synth.config_seed(4, 6), (K, M) if op_a else (M, K), np.int32, -100, 100)
    b = synth.integers(synth.config_seed(4, 7), (N, K) if op_b else (K, N), np.int32, -100, 100)
    c = synth.integers(synth.config_seed(4, 8), (M, N), np.int32, -100, 100)
    want = _exact_int32(3, a.T if op_a else a, b.T if op_b else b, -2, c)
    context = wk.Context.initFromDeviceType(wk.DeviceType.all)
    pipeline = wk.Pipeline.init(context.command_queues[0])
    try:
        tensors = []
        for host in (a, b, c):
            t = wk.Tensor.alloc("i32", context, pipeline, host.shape)
            wk.memory.readFromBuffer(pipeline, t, host)
            tensors.append(t)
        A, B, C = tensors
        packed = wk.GemmPackedTensors.init(pipeline, C, K, True)
        assert packed.workspace_bytes > 0
        name = wk._capi.load().wk_gemm_variant_with_workspace(raw.dtype_id("i32"), op_a, op_b, M, N, K, A.row_pitch, B.row_pitch,
                                                        C.row_pitch, A.buffer, B.buffer, C.buffer, packed.workspace_bytes)
        assert name == b"mfma_i32_packed"
        wk.blas.gemm(pipeline, 3, A, op_a, B, op_b, -2, C, packed)
        got = np.empty((M, N), dtype=np.int32)
        wk.memory.writeToBuffer(pipeline, C, got)
        pipeline.waitAndCleanup()
        assert np.array_equal(got, want)
        # second call on the same handle (the workspace is reused) from the new C
        wk.blas.gemm(pipeline, None, A, op_a, B, op_b, None, C, packed)
        wk.memory.writeToBuffer(pipeline, C, got)
        pipeline.waitAndCleanup()
        assert np.array_equal(got, _exact_int32(None, a.T if op_a else a, b.T if op_b else b, None, c))
        packed.deinit(pipeline)
        for t in tensors:
            t.release(pipeline)
    finally:
        pipeline.deinit()
        context.deinit()


@pytest.mark.parametrize("dtype,shape", [("i8", (768, 640, 1024)), ("cf32", (256, 320, 256))])
def test_packed_tensors_keep_b_across_calls(dtype, shape):
    """GemmPackedTensors.keepB: B is packed by the first blas.gemm and stays packed while the same B
    tensor comes back; a changed B shows only after invalidateB() (so the stale product in between is
    the proof that the pack pass of B was skipped); another B tensor is packed without being asked."""
    import wekua_amd as wk
    from helpers import assert_gemm_close, gemm_operands
    M, N, K = shape
    a1, b1, c0 = gemm_operands(dtype, M, N, K, 0, 1, 61)
    a2, b2, _ = gemm_operands(dtype, M, N, K, 0, 1, 62)
    context = wk.Context.initFromDeviceType(wk.DeviceType.all)
    pipeline = wk.Pipeline.init(context.command_queues[0])
    try:
        A = wk.Tensor.alloc(dtype, context, pipeline, (M, K))
        B = wk.Tensor.alloc(dtype, context, pipeline, (N, K))
        B_other = wk.Tensor.alloc(dtype, context, pipeline, (N, K))
        C = wk.Tensor.alloc(dtype, context, pipeline, (M, N))
        packed = wk.GemmPackedTensors.init(pipeline, C, K, True)
        assert packed.workspace_bytes > 0
        packed.keepB(True)

        def product(b_tensor, a_host, b_host_expected):
            wk.blas.gemm(pipeline, None, A, 0, b_tensor, 1, None, C, packed)
            got = np.empty_like(c0)
            wk.memory.writeToBuffer(pipeline, C, got)
            pipeline.waitAndCleanup()
            want = oracle.gemm(dtype, None, a_host, 0, b_host_expected, 1, None, c0)
            assert_gemm_close(dtype, got, want, None, a_host, 0, b_host_expected, 1, None, c0, K, what=dtype)

        wk.memory.readFromBuffer(pipeline, A, a1)
        wk.memory.readFromBuffer(pipeline, B, b1)
        wk.memory.readFromBuffer(pipeline, B_other, b2)
        product(B, a1, b1)                       # packs A and B
        wk.memory.readFromBuffer(pipeline, A, a2)
        product(B, a2, b1)                       # packs A only
        wk.memory.readFromBuffer(pipeline, B, b2)
        product(B, a2, b1)                       # B changed behind the handle's back: still the kept form
        packed.invalidateB()
        product(B, a2, b2)
        wk.memory.readFromBuffer(pipeline, B, b1)
        product(B_other, a2, b2)                 # another tensor: packed afresh
        product(B, a2, b1)                       # and back
        # B released and another tensor created in its place (same shape: the allocators hand back the
        # same host object and device block more often than not): a different tensor, so it is packed
        # afresh although every address may match the kept one
        for _ in range(3):
            product(B, a2, b1)
            B.release(pipeline)
            B = wk.Tensor.alloc(dtype, context, pipeline, (N, K))
            wk.memory.readFromBuffer(pipeline, B, b2)
            product(B, a2, b2)
            wk.memory.readFromBuffer(pipeline, B, b1)
            packed.invalidateB()
        packed.keepB(False)
        wk.memory.readFromBuffer(pipeline, B, b2)
        product(B, a2, b2)                       # off: every call packs both, as the reference does
        packed.deinit(pipeline)
        for t in (A, B, B_other, C):
            t.release(pipeline)
    finally:
        pipeline.deinit()
        context.deinit()
