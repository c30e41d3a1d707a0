"""CPU restatement (numpy) of the reference's tensor support operations: transpose, random.uniform,
toComplex / toReal.

TEST INFRASTRUCTURE ONLY: imported by tests/ -- never by the product path.

Pin status
----------
* transpose, to_complex, to_real: pure data movement; the reference's tests assert the coordinate
  property result[..j..i..] == tensor[..i..j..] (src/tensor/transpose.zig:113-671) and fixed values
  (src/tensor/convertions/to_complex.zig:298-436, to_real.zig:345-433), which tests/ restate as data.
* uniform: the reference's tests are statistical (mean / standard deviation within 5 %, values inside
  the range, equal seeds equal, different seeds different: src/tensor/random/uniform.zig:215-833);
  tests/test_oracle_tensor_ops.py runs them on this restatement.  The exact bits of the hash are
  PARITY UNPINNED: the reference holds no golden value for it, and its formula is not the
  library xxHash it is modelled on (operator precedence in kernels/uniform.cl:52-53 changes it), so no
  published vector applies.  It is restated from the kernel text, including that the seed enters
  unmixed and that the two halves of the index trade places.
* The reference keys the hash on the element's index in ITS padded buffer; here it is the logical
  row-major index, which is the same number whenever the reference's tensor has no padding.
"""
from __future__ import annotations

import numpy as np

_M = np.uint64(0xFFFFFFFFFFFFFFFF)
_P = np.uint64(0x9FB21C651E98DF25)
_KEY0 = np.uint64(0x7C01812CF721AD1C ^ 0xDED46DE9839097DB)


def _rotl(x, k):
    return (x << np.uint64(k)) | (x >> np.uint64(64 - k))


def hash64(index, seed: int):
    """kernels/uniform.cl:31-55."""
    index = np.asarray(index, dtype=np.uint64)
    with np.errstate(over="ignore"):
        key = _KEY0 - np.uint64(seed)  # `seed ^ ((seed & 0xFFFFFFFF00000000) << 32)` is the seed itself
        combined = ((index & np.uint64(0xFFFFFFFF)) << np.uint64(32)) + (index >> np.uint64(32))
        x0 = combined ^ key
        x1 = x0 ^ _rotl(x0, 49) ^ (_rotl(x0, 24) * _P)
        x2 = x1 ^ (((x1 >> np.uint64(35)) + np.uint64(8)) * _P)
        return x2 ^ (x2 >> np.uint64(28))


def _component(h, sub: np.dtype, min_value, max_value):
    if min_value is not None or max_value is not None:
        info = np.finfo(sub) if sub.kind == "f" else np.iinfo(sub)
        mn = sub.type(min_value if min_value is not None else info.min)
        mx = sub.type(max_value if max_value is not None else info.max)
        if sub.kind == "f":
            rng = sub.type(mx - mn)
        else:
            rng = np.array(int(mx) - int(mn)).astype(np.dtype("u%d" % sub.itemsize)).view(sub)[()]  # wraps
        normalized = h.astype(np.float64) / 18446744073709551616.0
        val = np.float64(mn) + normalized * np.float64(rng)
        return val.astype(sub)  # float: round; integer: truncate toward zero
    if sub.kind == "f":
        return (h.astype(sub) / sub.type(18446744073709551616.0)).astype(sub)
    return h.astype(np.dtype("u%d" % sub.itemsize)).view(sub)


def uniform(dtype_name: str, shape, seed: int, min_value=None, max_value=None):
    """random.uniform over the logical elements (uniform.cl:57-180).  Complex dtypes ('c' + name)
    return a trailing (re, im) axis drawn from hash(2*index) and hash(2*index + 1)."""
    cplx = dtype_name.startswith("c")
    sub = np.dtype({"i8": np.int8, "u8": np.uint8, "i16": np.int16, "u16": np.uint16, "i32": np.int32, "u32": np.uint32,
                    "i64": np.int64, "u64": np.uint64, "f32": np.float32, "f64": np.float64}[dtype_name[1:] if cplx else dtype_name])
    n = int(np.prod(shape))
    idx = np.arange(n, dtype=np.uint64)
    if cplx:
        re = _component(hash64(idx << np.uint64(1), seed), sub, min_value, max_value)
        im = _component(hash64((idx << np.uint64(1)) + np.uint64(1), seed), sub, min_value, max_value)
        return np.stack([re, im], axis=-1).reshape(tuple(shape) + (2,))
    return _component(hash64(idx, seed), sub, min_value, max_value).reshape(shape)


def transpose(x, dim0: int, dim1: int):
    """src/tensor/kernels/transpose.cl: exchange two dimensions (a trailing (re, im) axis stays last)."""
    return np.ascontiguousarray(np.swapaxes(x, dim0, dim1))


def to_complex(src, dst, space: int):
    """convertions/kernels/to_complex.cl: writes src into component `space` of dst, keeps the other."""
    out = dst.copy()
    out[..., space] = src
    return out


def to_real(src, space: int):
    """convertions/kernels/to_real.cl."""
    return np.ascontiguousarray(src[..., space])
