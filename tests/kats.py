"""The reference's own known-answer cases for gemm and axpy, as data.

Each case is what one Zig `test` block of the reference asserts (src/blas/axpy.zig:178-972,
src/blas/gemm.zig:900-1307 with helpers src/blas/test_helpers.zig:38-247).  The same table
drives two suites: the CPU oracle (tests/test_oracle_kats.py) and the HIP path through the
reference-shaped API (tests/test_reference_kats_gpu.py).
"""
import numpy as np

import oracle

NN, T_ = 0, 1

# (m, k, op_a, op_b, alpha, beta) -- testGemmATimesIdentity calls, gemm.zig:957-1002 (cpu) and
# 1145-1185 (gpu); the packed suites (1066-1090, 1242-1270) reuse a subset with use_packing=true.
A_TIMES_IDENTITY = [
    (6, 10, NN, NN, None, None), (5, 7, NN, NN, None, None), (12, 20, NN, NN, None, None),
    (24, 8, NN, NN, None, None), (8, 24, NN, NN, None, None), (16, 48, NN, NN, None, None),
    (48, 16, NN, NN, None, None), (32, 96, NN, NN, None, None), (64, 128, NN, NN, None, None),
    (6, 10, NN, NN, 2, None), (12, 20, NN, NN, 2, None), (24, 8, NN, NN, 2, None), (16, 48, NN, NN, 2, None),
    (6, 10, NN, NN, 2, 3), (12, 20, NN, NN, 2, 3), (24, 8, NN, NN, 2, 3), (16, 48, NN, NN, 2, 3),
    (6, 10, T_, NN, None, None), (12, 20, T_, NN, None, None), (24, 8, T_, NN, None, None),
    (16, 48, T_, NN, None, None),
    (6, 10, NN, T_, None, None), (12, 20, NN, T_, None, None),
]
# (m, n, op_a, op_b, alpha, beta) -- testGemmIdentityTimesB calls, gemm.zig:969-975,1000-1002
IDENTITY_TIMES_B = [
    (10, 6, NN, NN, None, None), (7, 5, NN, NN, None, None), (20, 12, NN, NN, None, None),
    (8, 24, NN, NN, None, None), (48, 16, NN, NN, None, None), (96, 32, NN, NN, None, None),
    (128, 64, NN, NN, None, None),
    (10, 6, NN, T_, None, None), (20, 12, NN, T_, None, None), (8, 24, NN, T_, None, None),
]


def host_dtype(dtype):
    return oracle.real_np_dtype(dtype)


def iota(dtype, shape, start=1, scale=1):
    """makeDataValue (test_helpers.zig:38-44): element i holds i + 1 (complex: imaginary part 0)."""
    rd = host_dtype(dtype)
    n = int(np.prod(shape))
    vals = ((np.arange(n, dtype=np.int64) + start) * scale)
    if rd.kind in "iu":
        vals = vals.astype(np.uint64).astype(np.dtype("u%d" % rd.itemsize)).view(np.dtype("u%d" % rd.itemsize))
        vals = vals.astype(np.dtype("u%d" % rd.itemsize)).view(rd) if rd.kind == "i" else vals.astype(rd)
    else:
        vals = vals.astype(rd)
    vals = vals.reshape(shape)
    if oracle.is_complex(dtype):
        return np.stack([vals, np.zeros_like(vals)], axis=-1)
    return vals


def scalar(dtype, v):
    """A real test scalar as the dtype's element (complex: (v, 0)), None stays None."""
    if v is None:
        return None
    return (v, 0) if oracle.is_complex(dtype) else v


def expected_identity_product(dtype, data, transposed, alpha, beta):
    """computeExpected (test_helpers.zig:46-74): alpha*data (+ beta*1 when C was filled with ones)."""
    rd = host_dtype(dtype)
    cx = oracle.is_complex(dtype)
    d = data[..., 0] if cx else data
    d = d.T if transposed else d
    if rd.kind == "f":
        out = d.astype(rd) * rd.type(alpha if alpha is not None else 1)
        if beta is not None:
            out = out + rd.type(beta)
        out = out.astype(rd)
    else:
        bits = 8 * rd.itemsize
        mask = (1 << bits) - 1
        o = d.astype(object) * (alpha if alpha is not None else 1)
        if beta is not None:
            o = o + beta
        u = np.vectorize(lambda t: int(t) & mask, otypes=[object])(o)
        out = np.array(u, dtype=np.uint64).astype(np.dtype("u%d" % rd.itemsize)).view(rd).reshape(d.shape)
    if cx:
        return np.stack([out, np.zeros_like(out)], axis=-1)
    return np.ascontiguousarray(out)


def identity_matrix(dtype, n):
    rd = host_dtype(dtype)
    eye = np.eye(n, dtype=rd)
    if oracle.is_complex(dtype):
        return np.stack([eye, np.zeros_like(eye)], axis=-1)
    return eye


def ones(dtype, shape):
    rd = host_dtype(dtype)
    o = np.ones(shape, dtype=rd)
    if oracle.is_complex(dtype):
        return np.stack([o, np.zeros_like(o)], axis=-1)
    return o


# ---- axpy known answers (axpy.zig) ----------------------------------------------------------

def axpy_cases(dtype):
    """Yields (name, x, alpha, y, expected) for every axpy test block that applies to `dtype`."""
    rd = host_dtype(dtype)
    cx = oracle.is_complex(dtype)
    signed = rd.kind != "u"

    def mk(re, im=None):
        re = np.asarray(re).astype(rd)
        if not cx:
            return re
        im = np.zeros_like(re) if im is None else np.asarray(im).astype(rd)
        return np.stack([re, im], axis=-1)

    i5 = np.arange(5)
    # :178-283  y = 2*[1..5] + [10..50] = [12, 24, 36, 48, 60]
    yield ("basic", mk(i5 + 1), scalar(dtype, 2), mk((i5 + 1) * 10), mk((i5 + 1) * 2 + (i5 + 1) * 10))
    i4 = np.arange(4)
    # :285-385  alpha = null: [1..4] + [5..8]
    yield ("null_alpha", mk(i4 + 1), None, mk(i4 + 5), mk(2 * i4 + 6))
    # :387-502  alpha = -1 on signed types: [10,10,10,10] - [1..4] = [9, 8, 7, 6]
    if signed:
        yield ("minus_one", mk(i4 + 1), scalar(dtype, -1), mk(np.full(4, 10)), mk(10 - (i4 + 1)))
    # :504-617  2-D {2,3}: x = i (+ 2i*j), y = 3i (+ i*j), alpha = 3 -> real 6i, imag 7i
    i6 = np.arange(6).reshape(2, 3)
    if cx:
        yield ("2d", mk(i6, i6 * 2), (3, 0), mk(i6 * 3, i6), mk(i6 * 3 + i6 * 3, i6 * 2 * 3 + i6))
    else:
        yield ("2d", mk(i6), 3, mk(i6 * 3), mk(i6 * 3 + i6 * 3))
    # :619-678  3-D {2,2,2}: ones, fives, alpha = 2 -> sevens
    o8 = np.ones((2, 2, 2))
    yield ("3d", mk(o8), scalar(dtype, 2), mk(o8 * 5), mk(o8 * 7))
    # :817-876  zero alpha leaves y = 10
    o5 = np.ones(5)
    yield ("zero_alpha", mk(o5), scalar(dtype, 0), mk(o5 * 10), mk(o5 * 10))
    # :878-972  complex alpha (2 + i): x = (i+1)(1 + j), y = 2i + 3i*j
    if cx:
        i3 = np.arange(3)
        xr = xi = i3 + 1
        yield ("complex_alpha", mk(xr, xi), (2, 1), mk(i3 * 2, i3 * 3),
               mk((2 * xr - xi) + i3 * 2, (xr + 2 * xi) + i3 * 3))
