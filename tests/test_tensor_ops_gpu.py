"""GPU: the reference's tensor support operations through the mirrored API -- transpose,
memory.copy / getValue / putValue, random.uniform, toComplex / toReal, N-d identity -- restating the
reference's own test blocks (src/tensor/{transpose,identity}.zig, src/tensor/memory/main.zig,
src/tensor/random/uniform.zig, src/tensor/convertions/*.zig) and comparing with oracle/tensor_ops.py.
Everything here moves or generates data, so every comparison is exact, with one stated exception:
ranged random values are formed as min + h/2^64 * range in double on the device, where the
multiply-add may be fused, so integers may differ by one unit on rare elements and floats by a few
ulp of |min| + |range|."""
import numpy as np
import pytest

import oracle
import wekua_amd as wk
from oracle import tensor_ops as ot
from wekua_amd import Context, DeviceType, Pipeline, Space, Tensor, convertions, fill, identity, memory, random, transpose

pytestmark = pytest.mark.gpu
REAL = wk.DTYPE_NAMES[:10]
ALL = wk.DTYPE_NAMES


@pytest.fixture(scope="module")
def env():
    context = Context.initFromDeviceType(DeviceType.all)
    pipeline = Pipeline.init(context.command_queues[0])
    yield context, pipeline
    pipeline.deinit()
    context.deinit()


def host_values(dtype, shape, seed=1):
    """Distinct, exactly representable values (complex: trailing (re, im) axis)."""
    rd = oracle.real_np_dtype(dtype)
    n = int(np.prod(shape)) * (2 if oracle.is_complex(dtype) else 1)
    vals = (np.arange(n, dtype=np.int64) * 7 + seed) % 120
    return vals.astype(rd).reshape(tuple(shape) + ((2,) if oracle.is_complex(dtype) else ()))


def upload(context, pipeline, dtype, host):
    shape = host.shape[:-1] if oracle.is_complex(dtype) else host.shape
    t = Tensor.alloc(dtype, context, pipeline, shape)
    memory.readFromBuffer(pipeline, t, host)
    return t


def download(pipeline, t):
    out = np.empty(t.host_shape(), dtype=oracle.real_np_dtype(t.dtype))
    memory.writeToBuffer(pipeline, t, out)
    pipeline.waitAndCleanup()
    return out


def swapped(shape, d0, d1):
    s = list(shape)
    s[d0], s[d1] = s[d1], s[d0]
    return tuple(s)


# ---- transpose -----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("shape,d0,d1", [((3, 4), 0, 1), ((2, 3, 4), 0, 1), ((2, 3, 4), 1, 2), ((2, 3, 4), 0, 2),
                                         ((2, 3, 4, 5), 1, 3), ((2, 3, 4, 5), 0, 2), ((3, 4), 1, 0), ((5, 7), 1, 1)])
def test_transpose_reference_cases(env, dtype, shape, d0, d1):
    # transpose.zig:113-671: 2-D, 3-D over each pair, 4-D, reversed order of the two dims, equal dims = copy
    context, pipeline = env
    xh = host_values(dtype, shape)
    x = upload(context, pipeline, dtype, xh)
    r = Tensor.alloc(dtype, context, pipeline, swapped(shape, d0, d1))
    transpose(pipeline, r, x, d0, d1)
    assert np.array_equal(download(pipeline, r), ot.transpose(xh, d0, d1))
    assert np.array_equal(download(pipeline, x), xh)
    x.release(pipeline)
    r.release(pipeline)


@pytest.mark.parametrize("dtype", ["u8", "i16", "f32", "f64", "cf32", "cf64"])
@pytest.mark.parametrize("shape,d0,d1", [((1000, 777), 0, 1), ((64, 64), 0, 1), ((65, 1), 0, 1), ((1, 129), 0, 1),
                                         ((5, 130, 67), 1, 2), ((33, 9, 70), 0, 2), ((7, 40, 256), 0, 1),
                                         ((2048, 4096), 0, 1)])
def test_transpose_large_and_ragged(env, dtype, shape, d0, d1):
    if shape == (2048, 4096) and dtype not in ("f32", "cf64"):
        pytest.skip("one small and one large element size is enough at this size")
    context, pipeline = env
    rd = oracle.real_np_dtype(dtype)
    n = int(np.prod(shape)) * (2 if oracle.is_complex(dtype) else 1)
    xh = (np.arange(n, dtype=np.int64) % 251).astype(rd).reshape(tuple(shape) + ((2,) if oracle.is_complex(dtype) else ()))
    x = upload(context, pipeline, dtype, xh)
    r = Tensor.alloc(dtype, context, pipeline, swapped(shape, d0, d1))
    transpose(pipeline, r, x, d0, d1)
    assert np.array_equal(download(pipeline, r), ot.transpose(xh, d0, d1))
    x.release(pipeline)
    r.release(pipeline)


def test_transpose_errors(env):
    context, pipeline = env
    x = Tensor.alloc("f32", context, pipeline, (3, 4))
    cases = [((4, 3, 1), 0, 1, "UnqualTensorsDimension"), ((4, 3), 0, 2, "InvalidValue"), ((4, 4), 0, 1, "UnqualTensorsDimension"),
             ((3, 4), 0, 1, "InvalidValue")]
    for shape, d0, d1, name in cases:
        r = Tensor.alloc("f32", context, pipeline, shape)
        with pytest.raises(wk.WekuaError) as e:
            transpose(pipeline, r, x, d0, d1)
        assert e.value.name == name, (shape, d0, d1)
        r.release(pipeline)
    x.release(pipeline)


# ---- memory.copy / getValue / putValue -------------------------------------------------------------

@pytest.mark.parametrize("dtype", ALL)
def test_put_value_get_value(env, dtype):
    # memory/main.zig:20-329: 1-D, 2-D, 3-D, several values in one tensor, zeroed tensor, overwrite
    context, pipeline = env
    cplx = oracle.is_complex(dtype)
    rd = oracle.real_np_dtype(dtype)
    for shape, coords in (((10,), [(5,), (0,), (9,)]), ((4, 5), [(2, 3), (0, 0), (3, 4)]), ((2, 3, 4), [(1, 2, 3), (0, 0, 0), (1, 0, 2)])):
        t = Tensor.alloc(dtype, context, pipeline, shape)
        got = np.zeros(2 if cplx else 1, dtype=rd)
        memory.getValue(pipeline, t, coords[0], got)
        pipeline.waitAndCleanup()
        assert not got.any()  # alloc zero-fills
        want = {}
        for i, c in enumerate(coords):
            v = (42 + i, 7 + i) if cplx else 42 + i
            memory.putValue(pipeline, t, c, v)
            want[c] = v
        memory.putValue(pipeline, t, coords[0], (99, 1) if cplx else 99)  # overwrite
        want[coords[0]] = (99, 1) if cplx else 99
        full = download(pipeline, t)
        for c, v in want.items():
            memory.getValue(pipeline, t, c, got)
            pipeline.waitAndCleanup()
            assert np.array_equal(got, np.array(v if cplx else [v], dtype=rd)), (shape, c)
            assert np.array_equal(np.atleast_1d(full[c]), np.array(v if cplx else [v], dtype=rd))
        assert np.count_nonzero(full) == len(want) * (2 if cplx else 1)
        t.release(pipeline)


def test_put_get_value_invalid_coordinates(env):
    # memory/main.zig:331-377
    context, pipeline = env
    t = Tensor.alloc("f32", context, pipeline, (4, 5))
    one = np.zeros(1, np.float32)
    for coor in ((1,), (1, 2, 3), (4, 0), (0, 5)):
        with pytest.raises(wk.WekuaError) as e:
            memory.putValue(pipeline, t, coor, 1.0)
        assert e.value.name == "InvalidCoordinates"
        with pytest.raises(wk.WekuaError) as e:
            memory.getValue(pipeline, t, coor, one)
        assert e.value.name == "InvalidCoordinates"
    t.release(pipeline)


@pytest.mark.parametrize("dtype", ["i8", "f32", "cf64"])
@pytest.mark.parametrize("shape", [(7,), (5, 9), (3, 4, 6), (300, 4096)])
def test_memory_copy(env, dtype, shape):
    context, pipeline = env
    xh = host_values(dtype, shape, seed=3)
    src = upload(context, pipeline, dtype, xh)
    for vectors in (True, False):  # memory/copy.zig:84-98: same and different row pitch
        dst = Tensor.alloc(dtype, context, pipeline, shape, vectors)
        memory.copy(pipeline, src, dst)
        assert np.array_equal(download(pipeline, dst), xh)
        dst.release(pipeline)
    other = Tensor.alloc(dtype, context, pipeline, tuple(reversed(shape)) if len(shape) > 1 else (shape[0] + 1,))
    with pytest.raises(wk.WekuaError) as e:
        memory.copy(pipeline, src, other)
    assert e.value.name == "UnqualTensorsShape"
    other.release(pipeline)
    src.release(pipeline)


# ---- random.uniform ----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("shape", [(100,), (10, 10), (5, 6, 7), (3, 1000)])
def test_uniform_without_range_matches_the_restatement(env, dtype, shape):
    # uniform.zig:215-387
    context, pipeline = env
    t = Tensor.alloc(dtype, context, pipeline, shape)
    random.uniform(pipeline, t, 42)
    got = download(pipeline, t)
    want = ot.uniform(dtype, shape, 42)
    assert np.array_equal(got, want)
    if dtype[-3:] in ("f32", "f64"):
        assert got.min() >= 0.0 and got.max() <= 1.0
    t.release(pipeline)


@pytest.mark.parametrize("dtype", ALL)
def test_uniform_with_range(env, dtype):
    # uniform.zig:389-483, 764-833
    context, pipeline = env
    is_float = dtype[-3:] in ("f32", "f64")
    lo, hi = (-5.0, 5.0) if is_float else ((10, 100) if "u" in dtype else (-50, 50))
    t = Tensor.alloc(dtype, context, pipeline, (40, 50))
    random.uniform(pipeline, t, 7, lo, hi)
    got = download(pipeline, t)
    want = ot.uniform(dtype, (40, 50), 7, lo, hi)
    assert got.min() >= lo and got.max() <= hi
    if is_float:
        assert np.allclose(got, want, rtol=0, atol=4 * np.finfo(got.dtype).eps * (abs(lo) + abs(hi - lo)))
    else:
        diff = np.abs(got.astype(np.int64) - want.astype(np.int64))
        assert diff.max() <= 1 and np.count_nonzero(diff) <= got.size // 1000
    # only one bound given: the other is the type's extreme (uniform.zig:90-100)
    if is_float:
        random.uniform(pipeline, t, 7, 0.0, None)
        g2 = download(pipeline, t)
        assert g2.min() >= 0.0 and np.isfinite(g2).all() and g2.max() > 1e30
    t.release(pipeline)


@pytest.mark.parametrize("dtype", ["i32", "f32", "f64", "cf32"])
def test_uniform_statistics_and_seeds(env, dtype):
    # uniform.zig:485-762: same seed same values, other seed other values, mean and stddev within 5 %
    context, pipeline = env
    a = Tensor.alloc(dtype, context, pipeline, (10000,))
    b = Tensor.alloc(dtype, context, pipeline, (10000,))
    random.uniform(pipeline, a, 100)
    random.uniform(pipeline, b, 100)
    ga, gb = download(pipeline, a), download(pipeline, b)
    assert np.array_equal(ga, gb)
    random.uniform(pipeline, b, 200)
    assert not np.array_equal(ga, download(pipeline, b))
    random.uniform(pipeline, b, None)  # clock seed: just has to run
    if dtype != "i32":
        v = ga.astype(np.float64)
        assert abs(v.mean() - 0.5) < 0.05 and abs(v.std() - 0.289) < 0.05
    else:
        random.uniform(pipeline, a, 42, 0, 100)
        v = download(pipeline, a).astype(np.float64)
        assert abs(v.mean() - 50) < 5 and abs(v.std() - 100 / np.sqrt(12)) < 5
    a.release(pipeline)
    b.release(pipeline)


# ---- toComplex / toReal ------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", REAL)
@pytest.mark.parametrize("shape", [(6,), (3, 4), (2, 3, 4), (70, 130)])
def test_to_complex_and_to_real(env, dtype, shape):
    # to_complex.zig:100-656, to_real.zig:99-750: each space, combination, overwrite, round trip
    context, pipeline = env
    cd = "c" + dtype
    re_h, im_h = host_values(dtype, shape, seed=2), host_values(dtype, shape, seed=5)
    re_t, im_t = upload(context, pipeline, dtype, re_h), upload(context, pipeline, dtype, im_h)
    z = Tensor.alloc(cd, context, pipeline, shape)
    fill.constant(pipeline, z, (9, 9))
    convertions.toComplex(pipeline, re_t, z, Space.real)
    want = ot.to_complex(re_h, np.full(tuple(shape) + (2,), 9, dtype=re_h.dtype), 0)
    assert np.array_equal(download(pipeline, z), want)  # the other component is kept
    convertions.toComplex(pipeline, im_t, z, Space.imag)
    want = ot.to_complex(im_h, want, 1)
    assert np.array_equal(download(pipeline, z), want)
    out = Tensor.alloc(dtype, context, pipeline, shape)
    convertions.toReal(pipeline, z, out, Space.imag)
    assert np.array_equal(download(pipeline, out), im_h)
    convertions.toReal(pipeline, z, out, Space.real)  # overwrites the previous extraction
    assert np.array_equal(download(pipeline, out), re_h)
    bad = Tensor.alloc(cd, context, pipeline, tuple(s + 1 for s in shape))
    with pytest.raises(wk.WekuaError) as e:
        convertions.toComplex(pipeline, re_t, bad, Space.real)
    assert e.value.name == "UnqualTensorsShape"
    with pytest.raises(wk.WekuaError) as e:
        convertions.toReal(pipeline, bad, out, Space.real)
    assert e.value.name == "UnqualTensorsShape"
    for t in (re_t, im_t, z, out, bad):
        t.release(pipeline)


def test_to_complex_specific_values(env):
    # to_complex.zig:298-436: [1.5, 2.5, 3.5, 4.5] into real, [10, 20, 30, 40] into imag
    context, pipeline = env
    r = upload(context, pipeline, "f32", np.array([1.5, 2.5, 3.5, 4.5], np.float32))
    i = upload(context, pipeline, "f32", np.array([10, 20, 30, 40], np.float32))
    z = Tensor.alloc("cf32", context, pipeline, (4,))
    convertions.toComplex(pipeline, r, z, Space.real)
    convertions.toComplex(pipeline, i, z, Space.imag)
    assert np.array_equal(download(pipeline, z), np.array([[1.5, 10], [2.5, 20], [3.5, 30], [4.5, 40]], np.float32))
    for t in (r, i, z):
        t.release(pipeline)


# ---- identity in N dimensions ------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("shape", [(1, 1), (5, 5), (3, 3, 3), (2, 2, 2, 2), (7, 7, 7)])
def test_identity_nd(env, dtype, shape):
    # identity.zig:77-509: ones where all coordinates agree, zeros elsewhere, previous contents overwritten
    context, pipeline = env
    t = Tensor.alloc(dtype, context, pipeline, shape)
    fill.constant(pipeline, t, (5, 5) if oracle.is_complex(dtype) else 5)
    identity(pipeline, t)
    got = download(pipeline, t)
    want = np.zeros_like(got)
    for i in range(shape[0]):
        if oracle.is_complex(dtype):
            want[(i,) * len(shape) + (0,)] = 1
        else:
            want[(i,) * len(shape)] = 1
    assert np.array_equal(got, want)
    t.release(pipeline)


def test_identity_rejects_unequal_extents(env):
    context, pipeline = env
    for shape in ((3, 4), (3, 3, 4)):
        t = Tensor.alloc("f32", context, pipeline, shape)
        with pytest.raises(wk.WekuaError) as e:
            identity(pipeline, t)
        assert e.value.name == "InvalidValue"
        t.release(pipeline)
