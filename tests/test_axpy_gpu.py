"""GPU parity: wk_axpy (through the C ABI) against the oracle on the same seeded inputs."""
import numpy as np
import pytest

import oracle
from helpers import make_operand

pytestmark = pytest.mark.gpu

ALL_DTYPES = oracle.DTYPE_NAMES


def run_axpy(dev, dtype, x, alpha, y, pitched=False):
    cx = oracle.is_complex(dtype)
    shape = x.shape[:-1] if cx else x.shape
    cols = shape[-1]
    rows = shape[-2] if len(shape) >= 2 else 1
    depth = int(np.prod(shape[:-2])) if len(shape) >= 3 else 1
    tail = (2,) if cx else ()
    x3 = x.reshape((depth, rows, cols) + tail)
    y3 = y.reshape((depth, rows, cols) + tail)
    if pitched:
        if pitched == "aligned":  # row starts on 16-byte boundaries for every dtype: the vector row kernel
            xrp, yrp = (cols + 15) // 16 * 16 + 16, (cols + 15) // 16 * 16 + 32
        else:
            xrp, yrp = cols + 3, cols + 5
        xs = np.full((depth, rows + 1, xrp) + tail, 55, dtype=x.dtype)
        ys = np.full((depth, rows + 2, yrp) + tail, 66, dtype=y.dtype)
        xs[:, :rows, :cols] = x3
        ys[:, :rows, :cols] = y3
        xsp, ysp = (rows + 1) * xrp, (rows + 2) * yrp
    else:
        xs, ys = x3, y3
        xrp = yrp = cols
        xsp = ysp = rows * cols
    dx, dy = dev.upload(xs), dev.upload(ys)
    dev.axpy(dtype, (depth, rows, cols), dx, xrp, xsp, alpha, dy, yrp, ysp)
    dev.sync()
    out = dy.download(ys.dtype, ys.shape)
    dx.free(); dy.free()
    if pitched:
        mask = np.ones(out.shape, dtype=bool)
        mask[:, :rows, :cols] = False
        assert (out[mask] == 66).all(), "axpy wrote outside the logical region"
        out = np.ascontiguousarray(out[:, :rows, :cols])
    return out.reshape(y.shape)


def expect(dtype, x, alpha, y):
    """Integers: the exact result mod 2^w.  Floats: the fused form fma(alpha, x, y), which is
    what the HIP kernel computes and one of the two roundings the reference permits."""
    if oracle.is_float(dtype):
        return oracle.axpy(dtype, x, alpha, y, contract=True)
    want = oracle.axpy(dtype, x, alpha, y)
    # the C restatement must agree with exact arithmetic, except for the reference's own
    # quirk that a complex alpha of (-1, -1) is treated as a subtraction (axpy.zig:75-77)
    if not (oracle.is_complex(dtype) and alpha is not None and tuple(alpha) == (-1, -1)):
        assert np.array_equal(want, oracle.semantic_axpy(dtype, x, alpha, y))
    return want


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_axpy_all_dtypes_shapes_alphas(dev, dtype):
    signed = oracle.real_np_dtype(dtype).kind != "u"
    cx = oracle.is_complex(dtype)
    alphas = [None, 2, 0, 3]
    if signed:
        alphas.append(-1)
    if oracle.is_float(dtype):
        alphas += [0.75, -1.0 + 1e-9 if dtype.endswith("f64") else -1.0]
    if cx:
        alphas = [None, (2, 0), (2, 1), (0, 0)] + ([(-1, 0), (-1, -1)] if signed else [])
    for shape in [(1,), (5,), (4,), (2, 3), (2, 2, 2), (3, 5, 7), (1000,), (4099,), (65536 + 3,), (2, 3, 4, 5),
                  (4, 1, 5), (3, 1, 70), (2, 3, 1, 7)]:
        for alpha in alphas:
            x = make_operand(dtype, shape, 7)
            y = make_operand(dtype, shape, 8)
            got = run_axpy(dev, dtype, x, alpha, y)
            want = expect(dtype, x, alpha, y)
            if oracle.is_float(dtype) and cx:
                np.testing.assert_allclose(got, want, rtol=1e-5 if dtype.endswith("f32") else 1e-13,
                                           atol=1e-6 if dtype.endswith("f32") else 1e-14)
            else:
                assert np.array_equal(got, want), f"{dtype} shape={shape} alpha={alpha}"


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_axpy_aligned_pitched_rows(dev, dtype):
    """Rows with gaps between them whose starts are 16-byte aligned (the layout of every 2-D / 3-D
    Tensor): full vectors plus a per-row tail, nothing written into the gaps."""
    signed = oracle.real_np_dtype(dtype).kind != "u"
    cx = oracle.is_complex(dtype)
    for shape in [(3, 16), (5, 37), (2, 3, 70), (7, 1), (4, 300), (33, 1025)]:
        for alpha in ([None, (2, 1)] + ([(-1, 0)] if signed else []) if cx else [None, 3] + ([-1] if signed else [])):
            x = make_operand(dtype, shape, 19)
            y = make_operand(dtype, shape, 20)
            got = run_axpy(dev, dtype, x, alpha, y, pitched="aligned")
            want = expect(dtype, x, alpha, y)
            if oracle.is_float(dtype) and cx:
                np.testing.assert_allclose(got, want, rtol=1e-5 if dtype.endswith("f32") else 1e-13,
                                           atol=1e-6 if dtype.endswith("f32") else 1e-14)
            else:
                assert np.array_equal(got, want), f"{dtype} shape={shape} alpha={alpha}"


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("shape", [(4, 1, 5), (3, 1, 70), (2, 3, 1, 7), (5, 1, 1)])
def test_axpy_single_row_slices_with_padded_pitch(dev, dtype, shape):
    """Slices of one row whose slice pitch is the padded row pitch (what a Tensor of shape
    (4, 1, 5) looks like): the logical elements are not contiguous although every slice holds a
    single row, so the contiguous-stream kernel must not be taken.  Gaps keep their poison."""
    cx = oracle.is_complex(dtype)
    depth, cols = int(np.prod(shape[:-2])), shape[-1]
    tail = (2,) if cx else ()
    x = make_operand(dtype, shape, 41)
    y = make_operand(dtype, shape, 42)
    alpha = (2, 1) if cx else 3
    ve = max(1, 16 // (x.dtype.itemsize * (2 if cx else 1)))
    for pitch in ((cols + ve - 1) // ve * ve + ve, cols + 3):       # 16-byte aligned rows; odd pitch
        xs = np.full((depth, pitch) + tail, 55, dtype=x.dtype)
        ys = np.full((depth, pitch) + tail, 66, dtype=y.dtype)
        xs[:, :cols] = x.reshape((depth, cols) + tail)
        ys[:, :cols] = y.reshape((depth, cols) + tail)
        dx, dy = dev.upload(xs), dev.upload(ys)
        dev.axpy(dtype, (depth, 1, cols), dx, pitch, pitch, alpha, dy, pitch, pitch)
        dev.sync()
        out = dy.download(ys.dtype, ys.shape)
        dx.free(); dy.free()
        assert (out[:, cols:] == 66).all(), "axpy wrote into the padding of a single-row slice"
        got = np.ascontiguousarray(out[:, :cols]).reshape(y.shape)
        want = expect(dtype, x, alpha, y)
        if oracle.is_float(dtype) and cx:
            np.testing.assert_allclose(got, want, rtol=1e-5 if dtype.endswith("f32") else 1e-13,
                                       atol=1e-6 if dtype.endswith("f32") else 1e-14)
        else:
            assert np.array_equal(got, want), f"{dtype} shape={shape} pitch={pitch}"


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u8", "cf32", "ci16"])
def test_axpy_pitched_regions(dev, dtype):
    for shape in [(5,), (2, 3), (3, 5, 7), (4, 33, 65)]:
        x = make_operand(dtype, shape, 9)
        y = make_operand(dtype, shape, 10)
        alpha = (2, 1) if oracle.is_complex(dtype) else 3
        got = run_axpy(dev, dtype, x, alpha, y, pitched=True)
        want = expect(dtype, x, alpha, y)
        if dtype == "cf32":
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
        else:
            assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("n", [2 ** 20, 2 ** 24])
def test_axpy_config_sizes(dev, dtype, n):
    """Benchmark configuration 2 at the sizes the oracle finishes in seconds (2^28: see the property test)."""
    x = make_operand(dtype, (n,), 0x5EED0020)
    y = make_operand(dtype, (n,), 0x5EED0021)
    got = run_axpy(dev, dtype, x, 0.75, y)
    want = oracle.axpy(dtype, x, 0.75, y, contract=True)
    assert np.array_equal(got, want)
    # and within one rounding of the unfused form the reference may equally produce
    unfused = oracle.axpy(dtype, x, 0.75, y, contract=False)
    eps = np.finfo(oracle.real_np_dtype(dtype)).eps
    assert np.all(np.abs(got.astype(np.float64) - unfused) <= eps * (np.abs(0.75 * x.astype(np.float64)) + np.abs(got)))


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_axpy_full_size_roundtrip(dev, dtype):
    """n = 2^28 (config 2): y + a*x - a*x restores y exactly when a*x is exactly representable
    (x, y small integers, a = 0.75 -> 3x/4 exact for multiples of 4), a size-independent property."""
    n = 2 ** 28
    rd = oracle.real_np_dtype(dtype)
    rng = np.random.default_rng(3)
    x = (rng.integers(-64, 64, size=n) * 4).astype(rd)
    y = rng.integers(-1000, 1000, size=n).astype(rd)
    dx, dy = dev.upload(x), dev.upload(y)
    dev.axpy(dtype, (1, 1, n), dx, n, n, 0.75, dy, n, n)
    mid = dy.download(rd, (n,))
    assert np.array_equal(mid, y + rd.type(0.75) * x)
    dev.axpy(dtype, (1, 1, n), dx, n, n, -0.75, dy, n, n)
    back = dy.download(rd, (n,))
    assert np.array_equal(back, y)
    dx.free(); dy.free()


def test_axpy_invalid_arguments(dev):
    import ctypes
    buf = dev.malloc(1024)
    s3 = (ctypes.c_uint64 * 3)(1, 2, 8)
    z3 = (ctypes.c_uint64 * 3)(1, 0, 8)
    lib, p = dev.lib, buf.ptr
    assert lib.wk_axpy(dev.stream, 8, z3, p, 8, 16, p, 8, 16, None) == 1      # zero dim
    assert lib.wk_axpy(dev.stream, 8, s3, p, 4, 16, p, 8, 16, None) == 1      # pitch < cols
    assert lib.wk_axpy(dev.stream, 25, s3, p, 8, 16, p, 8, 16, None) == 9     # bad dtype
    assert lib.wk_axpy(dev.stream, 8, s3, None, 8, 16, p, 8, 16, None) == 1   # null
    r1 = (ctypes.c_uint64 * 3)(2, 1, 8)
    assert lib.wk_axpy(dev.stream, 8, r1, p, 0, 4, p, 8, 8, None) == 1        # slice pitch < row of one-row slices
    buf.free()


@pytest.mark.parametrize("shape", [(70001, 24), (66000, 2, 8), (3, 66001, 4)])
def test_axpy_pitched_rows_beyond_grid_limits(dev, shape):
    """More rows or slices than one grid dimension holds (65535): the pitched-row kernel walks the
    rest in a loop."""
    x = make_operand("f32", shape, 29)
    y = make_operand("f32", shape, 30)
    got = run_axpy(dev, "f32", x, 0.75, y, pitched="aligned")
    assert np.array_equal(got, expect("f32", x, 0.75, y))
    gi = run_axpy(dev, "i16", make_operand("i16", shape, 31), -3, make_operand("i16", shape, 32), pitched="aligned")
    assert np.array_equal(gi, expect("i16", make_operand("i16", shape, 31), -3, make_operand("i16", shape, 32)))
