"""Shared helpers for the parity tests: seeded operands and the comparison rules.

Comparison bar:
  * integer dtypes (real and complex): bit-exact;
  * f32 / f64: |got - want| <= tol * sum_k |a||b| scaled by |alpha| (+ |beta||c|) with
    tol = 1e-5*sqrt(K) (f32) or 1e-12*sqrt(K) (f64) -- the tolerance the task states.
"""
import numpy as np

import oracle
from wekua_amd import synth

F32_TOL = 1e-5
F64_TOL = 1e-12


def make_operand(dtype: str, shape, seed: int, int_range=None) -> np.ndarray:
    rd = oracle.real_np_dtype(dtype)
    full = tuple(shape) + ((2,) if oracle.is_complex(dtype) else ())
    if rd.kind == "f":
        return synth.uniform(seed, full, rd)
    if int_range is None:
        info = np.iinfo(rd)
        lo, hi = int(info.min), int(info.max)
        if hi - lo + 1 > 2 ** 63:          # 64-bit: draw raw bits
            return synth.splitmix64(seed, int(np.prod(full))).view(np.int64).astype(rd).reshape(full)
    else:
        lo, hi = int_range
    return synth.integers(seed, full, rd, lo, hi)


def gemm_operands(dtype, M, N, K, op_a, op_b, seed, int_range=None):
    a = make_operand(dtype, (K, M) if op_a else (M, K), seed, int_range)
    b = make_operand(dtype, (N, K) if op_b else (K, N), seed + 1, int_range)
    c = make_operand(dtype, (M, N), seed + 2, int_range)
    return a, b, c


def assert_gemm_close(dtype, got, want, alpha, a, op_a, b, op_b, beta, c, K, what=""):
    rd = oracle.real_np_dtype(dtype)
    if rd.kind != "f":
        if not np.array_equal(got, want):
            bad = np.argwhere(got != want)
            raise AssertionError(f"{what}: {len(bad)} integer mismatches, first at {bad[0]}: "
                                 f"got {got[tuple(bad[0])]} want {want[tuple(bad[0])]}")
        return
    tol = (F32_TOL if rd.itemsize == 4 else F64_TOL) * np.sqrt(K)
    bound = oracle.gemm_abs_bound(dtype, alpha, a, op_a, b, op_b, beta, c)
    if oracle.is_complex(dtype):
        bound = bound[..., None]
    err = np.abs(got.astype(np.float64) - want.astype(np.float64)) / np.maximum(bound, 1e-300)
    worst = float(err.max())
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    assert worst <= tol, f"{what}: relative error {worst:.3e} > {tol:.3e}"
