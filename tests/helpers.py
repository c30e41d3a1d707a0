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


def gemm_bound_fast(dtype, alpha, a, op_a, b, op_b, beta, c):
    """|alpha| (|op(A)| |op(B)|) + |beta| |C| for the large real float cases, the product taken in the
    operands' own precision (it is only the scale the errors are measured against: a relative
    error of 1e-4 in it moves nothing) so that an 8192^3 case costs one sgemm, not one dgemm."""
    A, B = np.abs(a), np.abs(b)
    A = A.T if op_a else A
    B = B.T if op_b else B
    out = (A @ B).astype(np.float64)
    out *= 1.0 if alpha is None else abs(float(alpha))
    if beta is not None:
        out += abs(float(beta)) * np.abs(c)
    return out


def gemm_errors_everywhere(dtype, got, want, bound, K):
    """Relative error of every entry (in units of the tolerance): |got - want| / (tol * bound)."""
    rd = oracle.real_np_dtype(dtype)
    tol = (F32_TOL if rd.itemsize == 4 else F64_TOL) * np.sqrt(K)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    err /= np.maximum(bound, 1e-300)
    err /= tol
    return err


def assert_every_entry(dtype, got, want, bound, K, what=""):
    """Entry-by-entry comparison of a whole product, with the first bad 32x32 block named."""
    assert got.shape == want.shape
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = gemm_errors_everywhere(dtype, got, want, bound, K)
    worst = float(err.max())
    if worst > 1.0:
        i, j = np.unravel_index(int(err.argmax()), err.shape)
        bad = np.argwhere(err > 1.0)
        blocks = sorted({(int(r) // 32, int(c) // 32) for r, c in bad[:4096]})
        raise AssertionError(f"{what}: {len(bad)} entries beyond the tolerance, worst {worst:.3g} x tol at ({i}, {j}): "
                             f"got {got[i, j]!r} want {want[i, j]!r}; 32x32 blocks hit (first few): {blocks[:8]}")


def lattice_points(M, N, block=32, ragged_edges=True):
    """One entry in every `block` x `block` block of an M x N matrix, at a position inside the block that
    walks through all block*block positions as the block index advances (so that over 1024 blocks every
    lane x accumulator-register slot of a 32x32 matrix-instruction block has been looked at), plus the
    whole last row and last column (where ragged shapes keep their partial tiles)."""
    bi = np.arange((M + block - 1) // block)
    bj = np.arange((N + block - 1) // block)
    BI, BJ = np.meshgrid(bi, bj, indexing="ij")
    slot = (BI * 37 + BJ * 101 + (BI // block) * 5 + (BJ // block) * 331) % (block * block)
    ii = np.minimum(BI * block + slot // block, M - 1).ravel()
    jj = np.minimum(BJ * block + slot % block, N - 1).ravel()
    if ragged_edges:
        ii = np.concatenate([ii, np.full(N, M - 1), np.arange(M)])
        jj = np.concatenate([jj, np.arange(N), np.full(M, N - 1)])
    return ii, jj


def lattice_errors(dtype, got, alpha, a, op_a, b, op_b, beta, c, K, block=32):
    """float64 dot products at the lattice points, block row by block row.  Returns (ii, jj, err) with err in
    units of the tolerance."""
    rd = oracle.real_np_dtype(dtype)
    tol = (F32_TOL if rd.itemsize == 4 else F64_TOL) * np.sqrt(K)
    A = a.T if op_a else a
    B = b.T if op_b else b
    M, N = got.shape
    ii, jj = lattice_points(M, N, block)
    al = 1.0 if alpha is None else float(alpha)
    err = np.empty(len(ii))
    order = np.argsort(ii, kind="stable")
    ii, jj = ii[order], jj[order]
    start = 0
    while start < len(ii):
        stop = min(start + 4096, len(ii))
        Ar = A[ii[start:stop]].astype(np.float64)
        Bc = B[:, jj[start:stop]].astype(np.float64).T
        want = al * np.einsum("ik,ik->i", Ar, Bc)
        bound = abs(al) * np.einsum("ik,ik->i", np.abs(Ar), np.abs(Bc))
        if beta is not None:
            c0 = c[ii[start:stop], jj[start:stop]].astype(np.float64)
            want += float(beta) * c0
            bound += abs(float(beta)) * np.abs(c0)
        err[start:stop] = np.abs(got[ii[start:stop], jj[start:stop]].astype(np.float64) - want) / (tol * np.maximum(bound, 1e-300))
        start = stop
    return ii, jj, err
