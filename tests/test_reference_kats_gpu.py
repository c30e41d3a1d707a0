"""GPU: the reference's own test blocks (src/blas/axpy.zig:178-972, src/blas/gemm.zig:900-1307),
re-stated against the reference-shaped API of wekua_amd.  Every assertion is exact equality,
as in the Zig tests.  Integers run the identity products too (the reference restricts those to
float types; A*I is exact in every ring)."""
import numpy as np
import pytest

import kats
import oracle
import wekua_amd as wk
from wekua_amd import Context, DeviceType, Pipeline, Tensor, blas, fill, identity, memory

pytestmark = pytest.mark.gpu
Op = blas.Operation


@pytest.fixture(scope="module")
def env():
    context = Context.initFromDeviceType(DeviceType.all)
    pipeline = Pipeline.init(context.command_queues[0])
    yield context, pipeline
    pipeline.deinit()
    context.deinit()


def upload(context, pipeline, dtype, host, vectors_enabled=True):
    shape = host.shape[:-1] if oracle.is_complex(dtype) else host.shape
    t = Tensor.alloc(dtype, context, pipeline, shape, vectors_enabled)
    memory.readFromBuffer(pipeline, t, host)
    return t


def download(pipeline, t):
    out = np.empty(t.host_shape(), dtype=oracle.real_np_dtype(t.dtype))
    memory.writeToBuffer(pipeline, t, out)
    pipeline.waitAndCleanup()
    return out


# ------------------------------------------------------------------------------------ axpy ---

@pytest.mark.parametrize("dtype", wk.DTYPE_NAMES)
def test_axpy_reference_known_answers(env, dtype):
    context, pipeline = env
    for name, x_h, alpha, y_h, want in kats.axpy_cases(dtype):
        x = upload(context, pipeline, dtype, x_h)
        y = upload(context, pipeline, dtype, y_h)
        blas.axpy(pipeline, x, alpha, y)
        got = download(pipeline, y)
        assert np.array_equal(got, want), f"{dtype} {name}"
        x.release(pipeline)
        y.release(pipeline)


@pytest.mark.parametrize("dtype", wk.DTYPE_NAMES[:10])
def test_axpy_with_different_vector_configurations(env, dtype):
    """axpy.zig:680-761: tensors created with and without vectors give the same result."""
    context, pipeline = env
    x_h = kats.iota(dtype, (2, 3))
    y_h = kats.iota(dtype, (2, 3), scale=10)
    outs = []
    for ve in (True, False):
        x = upload(context, pipeline, dtype, x_h, ve)
        y = upload(context, pipeline, dtype, y_h, ve)
        blas.axpy(pipeline, x, 2, y)
        outs.append(download(pipeline, y))
        x.release(pipeline)
        y.release(pipeline)
    assert np.array_equal(outs[0], outs[1])
    assert np.array_equal(outs[0], kats.iota(dtype, (2, 3), scale=12))


@pytest.mark.parametrize("dtype", ["f32", "f64", "i8", "u16", "i64", "cf32", "ci32"])
@pytest.mark.parametrize("shape", [(4, 1, 5), (3, 1, 70), (2, 3, 1, 7)])
def test_axpy_tensors_whose_slices_hold_one_padded_row(env, dtype, shape):
    """Tensors with a row count of one and several slices: the row pitch is padded, so slices are
    not back to back.  Every logical element must be updated and none skipped."""
    context, pipeline = env
    x_h = kats.iota(dtype, shape)
    y_h = kats.iota(dtype, shape, scale=10)
    x = upload(context, pipeline, dtype, x_h)
    y = upload(context, pipeline, dtype, y_h)
    blas.axpy(pipeline, x, kats.scalar(dtype, 2), y)
    assert np.array_equal(download(pipeline, y), kats.iota(dtype, shape, scale=12))
    assert np.array_equal(download(pipeline, x), x_h)
    x.release(pipeline)
    y.release(pipeline)


def test_axpy_incompatible_tensor_shapes(env):
    """axpy.zig:763-815"""
    context, pipeline = env
    x = Tensor.alloc("f32", context, pipeline, (2, 3))
    y = Tensor.alloc("f32", context, pipeline, (2, 4))
    z = Tensor.alloc("f32", context, pipeline, (2, 3, 4))
    with pytest.raises(wk.WekuaError) as e:
        blas.axpy(pipeline, x, 2.0, y)
    assert e.value.name == "UnqualTensorsShape"
    with pytest.raises(wk.WekuaError) as e:
        blas.axpy(pipeline, x, 1.0, z)
    assert e.value.name == "UnqualTensorsShape"
    for t in (x, y, z):
        t.release(pipeline)


# ------------------------------------------------------------------------------------ gemm ---

def test_gemm_invalid_shapes(env):
    """gemm.zig:900-941"""
    context, pipeline = env
    a = Tensor.alloc("f32", context, pipeline, (2, 3))
    b = Tensor.alloc("f32", context, pipeline, (4, 5))
    c = Tensor.alloc("f32", context, pipeline, (2, 5))
    with pytest.raises(wk.WekuaError) as e:
        blas.gemm(pipeline, None, a, Op.no_transpose, b, Op.no_transpose, None, c, None)
    assert e.value.name == "InvalidValue"
    a3 = Tensor.alloc("f32", context, pipeline, (2, 3, 4))
    b2 = Tensor.alloc("f32", context, pipeline, (2, 3))
    c2 = Tensor.alloc("f32", context, pipeline, (2, 3))
    with pytest.raises(wk.WekuaError) as e:
        blas.gemm(pipeline, None, a3, Op.no_transpose, b2, Op.no_transpose, None, c2, None)
    assert e.value.name == "InvalidValue"
    for t in (a, b, c, a3, b2, c2):
        t.release(pipeline)


def test_gemm_tensors_of_different_contexts(env):
    """gemm.zig:450-452"""
    context, pipeline = env
    other = Context.initFromDeviceType(DeviceType.all)
    p2 = Pipeline.init(other.command_queues[0])
    a = Tensor.alloc("f32", context, pipeline, (4, 4))
    b = Tensor.alloc("f32", other, p2, (4, 4))
    c = Tensor.alloc("f32", context, pipeline, (4, 4))
    with pytest.raises(wk.WekuaError) as e:
        blas.gemm(pipeline, None, a, Op.no_transpose, b, Op.no_transpose, None, c, None)
    assert e.value.name == "UnqualTensorsContext"
    a.release(pipeline); c.release(pipeline); b.release(p2)
    p2.deinit(); other.deinit()


def a_times_identity(context, pipeline, dtype, m, k, op_a, op_b, use_packing, alpha, beta):
    """testGemmATimesIdentity, test_helpers.zig:88-165"""
    a_h = kats.iota(dtype, (k, m) if op_a else (m, k))
    a = upload(context, pipeline, dtype, a_h)
    ident = Tensor.alloc(dtype, context, pipeline, (k, k))
    c = Tensor.alloc(dtype, context, pipeline, (m, k))
    identity(pipeline, ident)
    if beta is not None:
        fill.one(pipeline, c)
    packed = blas.GemmPackedTensors.init(pipeline, c, k, True) if use_packing else None
    blas.gemm(pipeline, kats.scalar(dtype, alpha), a, op_a, ident, op_b, kats.scalar(dtype, beta), c, packed)
    got = download(pipeline, c)
    if packed:
        packed.deinit(pipeline)
    for t in (a, ident, c):
        t.release(pipeline)
    want = kats.expected_identity_product(dtype, a_h, bool(op_a), alpha, beta)
    assert np.array_equal(got, want), (dtype, m, k, op_a, op_b, use_packing, alpha, beta)


def identity_times_b(context, pipeline, dtype, m, n, op_a, op_b, use_packing, alpha, beta):
    """testGemmIdentityTimesB, test_helpers.zig:170-247"""
    b_h = kats.iota(dtype, (n, m) if op_b else (m, n))
    b = upload(context, pipeline, dtype, b_h)
    ident = Tensor.alloc(dtype, context, pipeline, (m, m))
    c = Tensor.alloc(dtype, context, pipeline, (m, n))
    identity(pipeline, ident)
    if beta is not None:
        fill.one(pipeline, c)
    packed = blas.GemmPackedTensors.init(pipeline, c, m, True) if use_packing else None
    blas.gemm(pipeline, kats.scalar(dtype, alpha), ident, op_a, b, op_b, kats.scalar(dtype, beta), c, packed)
    got = download(pipeline, c)
    if packed:
        packed.deinit(pipeline)
    for t in (b, ident, c):
        t.release(pipeline)
    want = kats.expected_identity_product(dtype, b_h, bool(op_b), alpha, beta)
    assert np.array_equal(got, want), (dtype, m, n, op_a, op_b, use_packing, alpha, beta)


@pytest.mark.parametrize("use_packing", [False, True])
@pytest.mark.parametrize("dtype", wk.DTYPE_NAMES)
def test_gemm_all_algorithms(env, dtype, use_packing):
    """gemm.zig:945-1307: A*I and I*B over the reference's size list, alpha/beta, transposes,
    with and without GemmPackedTensors."""
    context, pipeline = env
    small = oracle.real_np_dtype(dtype).itemsize == 1
    for (m, k, op_a, op_b, alpha, beta) in kats.A_TIMES_IDENTITY:
        if small and m * k > 120:
            continue
        a_times_identity(context, pipeline, dtype, m, k, op_a, op_b, use_packing, alpha, beta)
    for (m, n, op_a, op_b, alpha, beta) in kats.IDENTITY_TIMES_B:
        if small and m * n > 120:
            continue
        identity_times_b(context, pipeline, dtype, m, n, op_a, op_b, use_packing, alpha, beta)


def test_packed_tensors_validation(env):
    """gemm.zig:77-97 (init needs a 2-D result) and :250-270 (pack validates operand shapes)."""
    context, pipeline = env
    c3 = Tensor.alloc("f32", context, pipeline, (2, 3, 4))
    with pytest.raises(wk.WekuaError) as e:
        blas.GemmPackedTensors.init(pipeline, c3, 4, True)
    assert e.value.name == "InvalidValue"
    a = Tensor.alloc("f32", context, pipeline, (6, 10))
    b = Tensor.alloc("f32", context, pipeline, (10, 8))
    c = Tensor.alloc("f32", context, pipeline, (6, 8))
    pt = blas.GemmPackedTensors.init(pipeline, c, 10, True)
    pt.pack(pipeline, a, Op.no_transpose, b, Op.no_transpose)
    with pytest.raises(wk.WekuaError) as e:
        pt.pack(pipeline, a, Op.transpose, b, Op.no_transpose)
    assert e.value.name == "InvalidValue"
    bad = blas.GemmPackedTensors.init(pipeline, c, 11, True)
    with pytest.raises(wk.WekuaError):
        blas.gemm(pipeline, None, a, Op.no_transpose, b, Op.no_transpose, None, c, bad)
    pt.deinit(pipeline); bad.deinit(pipeline)
    for t in (a, b, c, c3):
        t.release(pipeline)


# ----------------------------------------------------------------------- tensor / pipeline ---

def test_tensor_layout_and_errors(env):
    context, pipeline = env
    with pytest.raises(wk.WekuaError) as e:
        Tensor.alloc("f32", context, pipeline, ())
    assert e.value.name == "InvalidValue"
    with pytest.raises(wk.WekuaError) as e:
        Tensor.alloc("f32", context, pipeline, (3, 0))       # tensor/main.zig:137
    assert e.value.name == "InvalidValue"
    t = Tensor.alloc("f32", context, pipeline, (5, 7))
    assert t.shape == (5, 7) and t.number_of_elements_without_padding == 35
    assert t.row_pitch == 8 and t.row_pitch % 4 == 0 and t.slice_pitch == 40 and t.size == 160
    assert t.vectors_enabled and t.pitches == (8, 1)
    with pytest.raises(wk.WekuaError) as e:                   # read_from_buffer.zig:19-21
        memory.readFromBuffer(pipeline, t, np.zeros(34, np.float32))
    assert e.value.name == "InvalidBuffer"
    # Tensor.alloc zero-fills, padding included (tensor/main.zig:274)
    assert not download(pipeline, t).any()
    d = Tensor.alloc("f64", context, pipeline, (2, 3, 5), vectors_enabled=False)
    assert d.row_pitch == 5 and d.slice_pitch == 15 and d.pitches == (15, 5, 1) and not d.vectors_enabled
    cx = Tensor.alloc("cf32", context, pipeline, (3, 3))
    assert not cx.vectors_enabled
    host = kats.iota("f32", (5, 7))
    memory.readFromBuffer(pipeline, t, host)
    assert np.array_equal(download(pipeline, t), host)         # pitched round trip
    for x in (t, d, cx):
        x.release(pipeline)


def test_identity_requires_equal_dims(env):
    context, pipeline = env
    t = Tensor.alloc("f32", context, pipeline, (3, 4))
    with pytest.raises(wk.WekuaError) as e:                   # identity.zig:21-26
        identity(pipeline, t)
    assert e.value.name == "InvalidValue"
    c = Tensor.alloc("i32", context, pipeline, (3, 3, 3))
    identity(pipeline, c)
    got = download(pipeline, c)
    want = np.zeros((3, 3, 3), np.int32)
    for i in range(3):
        want[i, i, i] = 1
    assert np.array_equal(got, want)
    t.release(pipeline); c.release(pipeline)


def test_pipeline_bookkeeping(env):
    """pipeline.zig:35-61: prevEvents is the last appended batch; waitAndCleanup empties it."""
    context, _ = env
    p = Pipeline.init(context.command_queues[0])
    assert p.prevEvents() == 0 and p.pending() == 0
    t = Tensor.alloc("f32", context, p, (4, 4))               # alloc enqueues the zero fill
    assert p.pending() == 1 and p.prevEvents() == 1
    fill.one(p, t)
    assert p.pending() == 2 and p.prevEvents() == 1
    p.waitAndCleanup()
    assert p.pending() == 0 and p.prevEvents() == 0
    p.waitAndCleanup()                                         # no-op on an empty pipeline
    t.release(p)
    p.deinit()


def test_context_cpu_device_type_is_unavailable():
    """The reference's CPU suites start with `initFromBestDevice(.cpu) catch return` (gemm.zig:947):
    asking for a CPU device is an error here too, never a silent host fallback."""
    with pytest.raises(wk.WekuaError) as e:
        Context.initFromBestDevice(DeviceType.cpu)
    assert e.value.name == "DevicesArrayEmpty"
