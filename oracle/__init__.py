"""CPU oracle for wekua's gemm / axpy -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package, and only as the checker / the timed CPU baseline.  The GPU product path in
wekua_amd/ never touches it.

Two independent restatements live here:

* ``libwk_oracle.so`` (wk_oracle.c): follows the reference's OpenCL CPU kernels in their
  own order of operations (src/blas/kernels/gemm_nxn.cl, gemm_2x2.cl, gemm_pack.cl,
  axpy.cl; block choice from src/tensor/work_configuration.zig:110-193 and
  src/blas/gemm.zig:42-58).
* ``semantic_gemm`` / ``semantic_axpy`` (numpy / Python big integers): what the
  mathematics fixes -- the exact product reduced mod 2^w for integers, a float64 /
  long-double accumulation for floats.  These pin the C restatement.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libwk_oracle.so")

REAL_NAMES = ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64", "f32", "f64"]
DTYPE_NAMES = REAL_NAMES + ["c" + n for n in REAL_NAMES]
_NP_REAL = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64,
            np.float32, np.float64]


def dtype_id(name: str) -> int:
    return DTYPE_NAMES.index(name)


def is_complex(name: str) -> bool:
    return name.startswith("c")


def real_np_dtype(name: str):
    return np.dtype(_NP_REAL[dtype_id(name) % 10])


def is_float(name: str) -> bool:
    return name.endswith("f32") or name.endswith("f64")


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (oracle/Makefile)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        u64, vp, ci = ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int
        L.wko_dtype_size.restype = ctypes.c_size_t
        L.wko_dtype_size.argtypes = [ci]
        L.wko_tensor_layout.argtypes = [ctypes.POINTER(u64), ci, ci, u64, ci, vp]
        L.wko_default_block_cpu.argtypes = [u64, u64, u64, ctypes.c_size_t]
        L.wko_get_algorithm.argtypes = [ci, u64]
        L.wko_axpy.argtypes = [ci, ctypes.POINTER(u64), vp, u64, u64, vp, u64, u64, vp, ci]
        L.wko_axpy_threads.argtypes = [ci, ctypes.POINTER(u64), vp, u64, u64, vp, u64, u64, vp, ci, ci]
        L.wko_gemm.argtypes = [ci, ci, ci, u64, u64, u64, vp, vp, u64, vp, u64, vp, vp, u64,
                               u64, ci, ci, ci, ci]
        L.wko_gemm_block.argtypes = [ci, ci, ci, u64, u64, u64, u64, ci]
        L.wko_pack.argtypes = [ci, vp, u64, u64, u64, vp, u64, u64, ci, u64, ci]
        _lib = L
    return _lib


class Layout(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint64) for n in (
        "depth", "rows", "cols", "padded_rows", "row_pitch", "row_pitch_for_vectors",
        "slice_pitch", "number_of_elements", "number_of_elements_without_padding",
        "number_of_vectors")]


def tensor_layout(shape, dtype: str, vector_width: int = 1, vectors_enabled: bool = True) -> Layout:
    arr = (ctypes.c_uint64 * len(shape))(*shape)
    out = Layout()
    rc = lib().wko_tensor_layout(arr, len(shape), dtype_id(dtype), vector_width,
                                 int(vectors_enabled), ctypes.byref(out))
    if rc:
        raise ValueError("invalid shape")
    return out


def _scalar_buf(dtype: str, value):
    """Host bytes of one element of `dtype` (None -> NULL)."""
    if value is None:
        return None, None
    rd = real_np_dtype(dtype)
    if is_complex(dtype):
        if isinstance(value, complex):
            value = (value.real, value.imag)
        a = np.array([_wrap(value[0], rd), _wrap(value[1], rd)], dtype=rd)
    else:
        a = np.array([_wrap(value, rd)], dtype=rd)
    return a, a.ctypes.data_as(ctypes.c_void_p)


def _wrap(v, rd):
    if rd.kind in "iu":
        return np.array(int(v) & ((1 << (8 * rd.itemsize)) - 1), dtype=np.uint64).astype(
            np.dtype("u%d" % rd.itemsize)).view(rd)[()] if rd.kind == "i" else \
            np.array(int(v) & ((1 << (8 * rd.itemsize)) - 1), dtype=np.uint64).astype(rd)[()]
    return rd.type(v)


def _check(arr: np.ndarray, dtype: str, logical_ndim=None):
    rd = real_np_dtype(dtype)
    if arr.dtype != rd or not arr.flags.c_contiguous:
        raise TypeError(f"expected C-contiguous {rd} array for {dtype}, got {arr.dtype}")
    if is_complex(dtype) and arr.shape[-1] != 2:
        raise TypeError("complex arrays carry a trailing (re, im) axis of length 2")


def axpy(dtype: str, x: np.ndarray, alpha, y: np.ndarray, contract: bool = False) -> np.ndarray:
    """Returns alpha*x + y computed like src/blas/kernels/axpy.cl (scalar build)."""
    _check(x, dtype); _check(y, dtype)
    if x.shape != y.shape:
        raise ValueError("UnqualTensorsShape")
    shape = x.shape[:-1] if is_complex(dtype) else x.shape
    cols = shape[-1]
    rows = shape[-2] if len(shape) >= 2 else 1
    depth = int(np.prod(shape[:-2], dtype=np.uint64)) if len(shape) >= 3 else 1
    out = y.copy()
    s3 = (ctypes.c_uint64 * 3)(depth, rows, cols)
    _keep, ap = _scalar_buf(dtype, alpha)
    rc = lib().wko_axpy(dtype_id(dtype), s3, x.ctypes.data, cols, rows * cols,
                        out.ctypes.data, cols, rows * cols, ap, int(contract))
    if rc:
        raise RuntimeError(f"wko_axpy failed: {rc}")
    return out


def axpy_inplace(dtype: str, x: np.ndarray, alpha, y: np.ndarray, contract: bool = False, threads: int = 0) -> None:
    """y = alpha*x + y in place on contiguous arrays, the elements spread over `threads` host threads
    (0: all).  What a timed CPU baseline calls: no copy of y, one pass."""
    _check(x, dtype); _check(y, dtype)
    if x.shape != y.shape or not (x.flags.c_contiguous and y.flags.c_contiguous):
        raise ValueError("UnqualTensorsShape")
    shape = x.shape[:-1] if is_complex(dtype) else x.shape
    cols = shape[-1]
    rows = shape[-2] if len(shape) >= 2 else 1
    depth = int(np.prod(shape[:-2], dtype=np.uint64)) if len(shape) >= 3 else 1
    s3 = (ctypes.c_uint64 * 3)(depth, rows, cols)
    _keep, ap = _scalar_buf(dtype, alpha)
    rc = lib().wko_axpy_threads(dtype_id(dtype), s3, x.ctypes.data, cols, rows * cols,
                                y.ctypes.data, cols, rows * cols, ap, int(contract), threads)
    if rc:
        raise RuntimeError(f"wko_axpy_threads failed: {rc}")


def _mat_dims(a: np.ndarray, dtype: str):
    shp = a.shape[:-1] if is_complex(dtype) else a.shape
    if len(shp) != 2:
        raise ValueError("InvalidValue")
    return shp


def gemm(dtype: str, alpha, a: np.ndarray, op_a: int, b: np.ndarray, op_b: int, beta,
         c: np.ndarray, vector_width: int = 1, packed: bool = False, block: int = 0,
         contract: bool = False, threads: int = 0) -> np.ndarray:
    """Returns alpha*op(A)op(B) + beta*C in the reference CPU device's order of operations."""
    for m in (a, b, c):
        _check(m, dtype)
    (ar, ac), (br, bc), (M, N) = _mat_dims(a, dtype), _mat_dims(b, dtype), _mat_dims(c, dtype)
    am, ak = (ac, ar) if op_a else (ar, ac)
    bk, bn = (bc, br) if op_b else (br, bc)
    if am != M or bn != N or ak != bk:
        raise ValueError("InvalidValue")
    out = c.copy()
    _ka, ap = _scalar_buf(dtype, alpha)
    _kb, bp = _scalar_buf(dtype, beta)
    rc = lib().wko_gemm(dtype_id(dtype), int(op_a), int(op_b), M, N, ak, ap,
                        a.ctypes.data, ac, b.ctypes.data, bc, bp, out.ctypes.data, N,
                        vector_width, int(packed), block, int(contract), threads)
    if rc:
        raise RuntimeError(f"wko_gemm failed: {rc}")
    return out


def gemm_block(dtype: str, op_a: int, op_b: int, M: int, N: int, K: int,
               vector_width: int = 1, packed: bool = False) -> int:
    return lib().wko_gemm_block(dtype_id(dtype), op_a, op_b, M, N, K, vector_width, int(packed))


def pack(dtype: str, src: np.ndarray, tiles: int, ktiles: int, block: int,
         vector_width: int = 1, transpose: bool = False) -> np.ndarray:
    _check(src, dtype)
    rows, cols = _mat_dims(src, dtype)
    vw = 1 if is_complex(dtype) else vector_width
    shape = (tiles, ktiles, block * block * vw) + ((2,) if is_complex(dtype) else ())
    dst = np.zeros(shape, dtype=src.dtype)
    rc = lib().wko_pack(dtype_id(dtype), src.ctypes.data, rows, cols, cols, dst.ctypes.data,
                        tiles, ktiles, block, vw, int(transpose))
    if rc:
        raise RuntimeError(f"wko_pack failed: {rc}")
    return dst


# ------------------------------------------------------------------ semantic oracle ---

def _to_exact(a: np.ndarray, dtype: str):
    """Object array of Python ints (or complex pairs as two object arrays) / longdouble arrays."""
    if is_float(dtype):
        hp = np.longdouble
        if is_complex(dtype):
            return a[..., 0].astype(hp), a[..., 1].astype(hp)
        return a.astype(hp), None
    if is_complex(dtype):
        return a[..., 0].astype(object), a[..., 1].astype(object)
    return a.astype(object), None


def _from_exact(re, im, dtype: str) -> np.ndarray:
    rd = real_np_dtype(dtype)

    def conv(v):
        if rd.kind in "iu":
            bits = 8 * rd.itemsize
            u = np.vectorize(lambda t: int(t) & ((1 << bits) - 1), otypes=[object])(v)
            return np.array(u, dtype=np.uint64).astype(np.dtype("u%d" % rd.itemsize)).view(rd) \
                .reshape(v.shape)
        return v.astype(rd)

    if im is None:
        return conv(re)
    return np.stack([conv(re), conv(im)], axis=-1)


def _scalar_exact(dtype: str, v):
    if v is None:
        return None
    if is_complex(dtype):
        if isinstance(v, complex):
            v = (v.real, v.imag)
        re, im = v
    else:
        re, im = v, 0
    if is_float(dtype):
        rd = real_np_dtype(dtype)
        return np.longdouble(rd.type(re)), np.longdouble(rd.type(im))
    return int(re), int(im)


def semantic_gemm(dtype: str, alpha, a, op_a, b, op_b, beta, c) -> np.ndarray:
    """alpha*op(A)op(B) + beta*C: exact mod 2^w for integers, long-double for floats.

    Option semantics of src/blas/gemm.zig:500-501,591-602: both None overwrites C;
    alpha only scales; beta given -> (alpha or 1)*AB + beta*C_old.
    """
    are, aim = _to_exact(a, dtype)
    bre, bim = _to_exact(b, dtype)
    cre, cim = _to_exact(c, dtype)
    if op_a:
        are = are.T
        aim = aim.T if aim is not None else None
    if op_b:
        bre = bre.T
        bim = bim.T if bim is not None else None
    if aim is None:
        pre, pim = are.dot(bre), None
    else:
        pre = are.dot(bre) - aim.dot(bim)
        pim = are.dot(bim) + aim.dot(bre)
    al, be = _scalar_exact(dtype, alpha), _scalar_exact(dtype, beta)
    if al is None and be is not None:
        al = _scalar_exact(dtype, (1, 0) if is_complex(dtype) else 1)
    if al is not None:
        if pim is None:
            pre = pre * al[0]
        else:
            pre, pim = pre * al[0] - pim * al[1], pre * al[1] + pim * al[0]
    if be is not None:
        if pim is None:
            pre = pre + cre * be[0]
        else:
            pre = pre + cre * be[0] - cim * be[1]
            pim = pim + cre * be[1] + cim * be[0]
    return _from_exact(pre, pim, dtype)


def semantic_axpy(dtype: str, x, alpha, y) -> np.ndarray:
    xre, xim = _to_exact(x, dtype)
    yre, yim = _to_exact(y, dtype)
    al = _scalar_exact(dtype, alpha) if alpha is not None else _scalar_exact(
        dtype, (1, 0) if is_complex(dtype) else 1)
    if xim is None:
        return _from_exact(yre + xre * al[0], None, dtype)
    return _from_exact(yre + xre * al[0] - xim * al[1], yim + xre * al[1] + xim * al[0], dtype)


def gemm_abs_bound(dtype: str, alpha, a, op_a, b, op_b, beta, c) -> np.ndarray:
    """|alpha| * (|op(A)| |op(B)|) + |beta| |C| in float64: the scale float errors are relative to."""
    def mag(m):
        m = m.astype(np.float64)
        return np.hypot(m[..., 0], m[..., 1]) if is_complex(dtype) else np.abs(m)

    def smag(v):
        if v is None:
            return 1.0
        if is_complex(dtype):
            if isinstance(v, complex):
                return abs(v)
            return float(np.hypot(v[0], v[1]))
        return abs(float(v))

    A, B = mag(a), mag(b)
    A = A.T if op_a else A
    B = B.T if op_b else B
    out = smag(alpha) * (A @ B)
    if beta is not None:
        out = out + smag(beta) * mag(c)
    return out
