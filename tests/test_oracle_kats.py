"""CPU: pins the oracle (oracle/wk_oracle.c) against the reference's own known answers and
against what the mathematics fixes.  No GPU, no HIP library."""
import itertools

import numpy as np
import pytest

import kats
import oracle
from helpers import assert_gemm_close, gemm_operands

ALL = oracle.DTYPE_NAMES
# (vector_width, packed, contract): the scalar build, the AVX2-like 8-lane build, the 16-lane build
# (4x4 micro-kernel), packed and unpacked, fused and unfused
BUILDS = [(1, False, False), (1, True, False), (8, False, False), (8, True, False), (16, True, False),
          (4, True, True), (1, False, True)]


@pytest.mark.parametrize("dtype", ALL)
def test_axpy_reference_known_answers(dtype):
    for name, x, alpha, y, want in kats.axpy_cases(dtype):
        for contract in (False, True):
            got = oracle.axpy(dtype, x, alpha, y, contract=contract)
            assert np.array_equal(got, want), f"{dtype} {name}"


@pytest.mark.parametrize("dtype", ALL)
def test_gemm_identity_known_answers(dtype):
    """gemm.zig:945-1307 (the reference runs these for float types only; integers are covered
    here as well since A*I is exact in every ring)."""
    small = oracle.real_np_dtype(dtype).itemsize == 1
    for (m, k, op_a, op_b, alpha, beta) in kats.A_TIMES_IDENTITY:
        if small and m * k > 120:       # i + 1 must fit the 8-bit element
            continue
        a = kats.iota(dtype, (k, m) if op_a else (m, k))
        ident = kats.identity_matrix(dtype, k)
        c = kats.ones(dtype, (m, k)) if beta is not None else np.zeros_like(kats.ones(dtype, (m, k)))
        want = kats.expected_identity_product(dtype, a, bool(op_a), alpha, beta)
        for vw, packed, contract in BUILDS:
            got = oracle.gemm(dtype, kats.scalar(dtype, alpha), a, op_a, ident, op_b, kats.scalar(dtype, beta), c,
                              vector_width=vw, packed=packed, contract=contract)
            assert np.array_equal(got, want), (dtype, m, k, op_a, op_b, alpha, beta, vw, packed)
    for (m, n, op_a, op_b, alpha, beta) in kats.IDENTITY_TIMES_B:
        if small and m * n > 120:
            continue
        b = kats.iota(dtype, (n, m) if op_b else (m, n))
        ident = kats.identity_matrix(dtype, m)
        c = np.zeros_like(kats.ones(dtype, (m, n)))
        want = kats.expected_identity_product(dtype, b, bool(op_b), alpha, beta)
        for vw, packed, contract in BUILDS:
            got = oracle.gemm(dtype, kats.scalar(dtype, alpha), ident, op_a, b, op_b, kats.scalar(dtype, beta), c,
                              vector_width=vw, packed=packed, contract=contract)
            assert np.array_equal(got, want), (dtype, m, n, op_a, op_b, vw, packed)


@pytest.mark.parametrize("dtype", ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64", "ci16", "cu32", "ci64"])
def test_integer_gemm_is_the_exact_product_mod_2w(dtype):
    """Ring identity: whatever the order of accumulation, the result is the exact product reduced
    mod 2^w.  Full-range random entries overflow constantly; compared with Python big integers."""
    signed = oracle.real_np_dtype(dtype).kind == "i"
    for (M, N, K), (op_a, op_b) in itertools.product([(5, 7, 3), (17, 9, 33), (32, 48, 64)], [(0, 0), (0, 1), (1, 0), (1, 1)]):
        a, b, c = gemm_operands(dtype, M, N, K, op_a, op_b, seed=100)
        for alpha, beta in [(None, None), (3, None), (7, -5 if signed else 250), (None, 2)]:
            al, be = kats.scalar(dtype, alpha), kats.scalar(dtype, beta)
            if oracle.is_complex(dtype) and alpha is not None:
                al = (alpha, 2)
            want = oracle.semantic_gemm(dtype, al, a, op_a, b, op_b, be, c)
            for vw, packed, _ in BUILDS[:5]:
                got = oracle.gemm(dtype, al, a, op_a, b, op_b, be, c, vector_width=vw, packed=packed)
                assert np.array_equal(got, want), (dtype, M, N, K, op_a, op_b, alpha, beta, vw, packed)


@pytest.mark.parametrize("dtype", ["f32", "f64", "cf32", "cf64"])
def test_float_gemm_against_long_double_brute_force(dtype):
    for (M, N, K), (op_a, op_b) in itertools.product([(5, 7, 3), (33, 17, 65), (64, 40, 128)], [(0, 0), (0, 1), (1, 0), (1, 1)]):
        a, b, c = gemm_operands(dtype, M, N, K, op_a, op_b, seed=200)
        for alpha, beta in [(None, None), (1.5, None), (1.5, 0.5), (None, -0.25)]:
            al, be = kats.scalar(dtype, alpha), kats.scalar(dtype, beta)
            want = oracle.semantic_gemm(dtype, al, a, op_a, b, op_b, be, c)
            for vw, packed, contract in BUILDS:
                got = oracle.gemm(dtype, al, a, op_a, b, op_b, be, c, vector_width=vw, packed=packed, contract=contract)
                assert_gemm_close(dtype, got, want, al, a, op_a, b, op_b, be, c, K, what=f"{dtype} vw={vw} packed={packed}")


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_float_gemm_closed_forms(dtype):
    rd = oracle.real_np_dtype(dtype)
    # all-ones operands: every entry is exactly K
    M, N, K = 24, 40, 96
    got = oracle.gemm(dtype, None, np.ones((M, K), rd), 0, np.ones((K, N), rd), 0, None, np.zeros((M, N), rd), vector_width=8)
    assert np.array_equal(got, np.full((M, N), K, rd))
    # rank one: (u v^T) B = u (v^T B), integer-valued so every partial sum is exact
    rng = np.random.default_rng(5)
    u = rng.integers(-8, 8, (M, 1)).astype(rd)
    v = rng.integers(-8, 8, (1, K)).astype(rd)
    B = rng.integers(-8, 8, (K, N)).astype(rd)
    got = oracle.gemm(dtype, None, (u @ v).astype(rd), 0, B, 0, None, np.zeros((M, N), rd), vector_width=8, packed=True)
    assert np.array_equal(got, u @ (v @ B))
    # integer-valued floats below 2^24: exact, so it must equal the int64 product bit for bit
    A = rng.integers(-50, 50, (M, K)).astype(rd)
    got = oracle.gemm(dtype, 2, A, 1 - 1, B, 0, 3, np.ones((M, N), rd))
    assert np.array_equal(got, (2 * (A.astype(np.int64) @ B.astype(np.int64)) + 3).astype(rd))


def test_beta_given_reads_c_even_when_zero():
    """gemm.zig:598-602 with gemm_2x2.cl:257: alpha*acc + beta*C is evaluated as written."""
    a, b, c = gemm_operands("f32", 8, 8, 8, 0, 0, seed=1)
    c[:] = np.nan
    assert np.isnan(oracle.gemm("f32", 1.0, a, 0, b, 0, 0.0, c)).all()
    assert np.isfinite(oracle.gemm("f32", 1.0, a, 0, b, 0, None, c)).all()


def test_pack_layout_formula():
    """What the reference's pack tests assert (gemm.zig:1309-1951): packed[tile][ktile][row][col]
    holds src[tile*BS + row][ktile*BS*vw + col] (transposed: the two swapped), zero outside."""
    n = 8
    for dtype in ["f32", "f64", "i32", "cf32"]:
        src = kats.iota(dtype, (n, n))
        cx = oracle.is_complex(dtype)
        for bs, vw, transpose in itertools.product([2, 4, 8], [1, 2, 4], [False, True]):
            vw_eff = 1 if cx else vw
            tw = bs * vw_eff
            tiles, ktiles = n // bs, max(1, -(-n // tw))
            packed = oracle.pack(dtype, src, tiles, ktiles, bs, vw, transpose)
            for tr in range(tiles):
                for tc in range(ktiles):
                    for r in range(bs):
                        for cc in range(tw):
                            if transpose:
                                sr, sc = tc * tw + cc, tr * bs + r
                            else:
                                sr, sc = tr * bs + r, tc * tw + cc
                            got = packed[tr, tc, r * tw + cc]
                            if sr < n and sc < n:
                                assert np.array_equal(got, src[sr, sc])
                            else:
                                assert not np.any(got)


def test_tensor_layout_matches_hand_computed_cases():
    """src/tensor/main.zig:142-199 by hand."""
    L = oracle.tensor_layout
    # 1-D {5}, f32, vector width 8: row_pitch 5 -> 8 (one vector) -> 16 (even vector count); one padded second row
    l = L((5,), "f32", 8)
    assert (l.rows, l.padded_rows, l.row_pitch, l.row_pitch_for_vectors, l.slice_pitch, l.number_of_elements) == (1, 2, 16, 2, 32, 32)
    # 2-D {5,7}, scalar device: rows 5 -> 6, pitch 7 -> 8
    l = L((5, 7), "f32", 1)
    assert (l.padded_rows, l.row_pitch, l.slice_pitch, l.number_of_elements_without_padding) == (6, 8, 48, 35)
    # 2-D {6,10}, width 4: pitch 10 -> 12 (3 vectors) -> 16 (4 vectors)
    l = L((6, 10), "f32", 4)
    assert (l.padded_rows, l.row_pitch, l.row_pitch_for_vectors, l.number_of_vectors) == (6, 16, 4, 24)
    # complex never vectorises; 3-D {2,3,4}
    l = L((2, 3, 4), "cf32", 8)
    assert (l.depth, l.padded_rows, l.row_pitch, l.slice_pitch, l.number_of_elements) == (2, 4, 4, 16, 32)
    # vectors disabled by the caller
    l = L((3, 9), "f64", 4, vectors_enabled=False)
    assert (l.padded_rows, l.row_pitch) == (4, 10)


def test_block_selection_matches_hand_computed_cases():
    """work_configuration.zig:110-193 (.global branch) and gemm.zig:42-58."""
    lib = oracle.lib()
    # f32, 8 lanes: 16x16 tile of 8-float vectors = 8 KiB fits 16 KiB, 32x32 = 32 KiB does not
    assert lib.wko_default_block_cpu(512, 512, 8, 4) == 16
    # scalar f32: 64x64x4 B = 16 KiB fits exactly
    assert lib.wko_default_block_cpu(512, 512, 1, 4) == 64
    # f64 scalar: 64x64x8 = 32 KiB does not fit, 32x32x8 = 8 KiB does
    assert lib.wko_default_block_cpu(512, 512, 1, 8) == 32
    # dims divisible by 2 only
    assert lib.wko_default_block_cpu(6, 10, 1, 4) == 2
    assert lib.wko_default_block_cpu(12, 20, 1, 4) == 4
    # getAlgorithm: largest block <= default dividing k
    assert lib.wko_get_algorithm(16, 512) == 16
    assert lib.wko_get_algorithm(64, 24) == 8
    assert lib.wko_get_algorithm(16, 6) == 2
    # whole plan: 512^3 f32 on an 8-lane CPU device, packed: k = 512/8 = 64 vectors -> block 16
    assert oracle.gemm_block("f32", 0, 0, 512, 512, 512, 8, True) == 16
    assert oracle.gemm_block("f32", 0, 0, 512, 512, 512, 1, False) == 64


def test_axpy_float_fused_and_unfused_differ_by_at_most_one_rounding():
    rng = np.random.default_rng(1)
    for dtype in ("f32", "f64"):
        rd = oracle.real_np_dtype(dtype)
        x = rng.uniform(-1, 1, 4096).astype(rd)
        y = rng.uniform(-1, 1, 4096).astype(rd)
        fused = oracle.axpy(dtype, x, 0.75, y, contract=True)
        plain = oracle.axpy(dtype, x, 0.75, y, contract=False)
        exact = y.astype(np.longdouble) + np.longdouble(0.75) * x.astype(np.longdouble)
        eps = np.finfo(rd).eps
        assert np.all(np.abs(fused - exact) <= 0.5 * eps * np.abs(exact) + np.finfo(rd).tiny)
        assert np.all(np.abs(plain - exact) <= eps * (np.abs(exact) + np.abs(0.75 * x)))


def test_axpy_shape_mismatch_raises():
    with pytest.raises(ValueError):
        oracle.axpy("f32", np.zeros((2, 3), np.float32), 2.0, np.zeros((2, 4), np.float32))


@pytest.mark.parametrize("dtype", ["f32", "f64", "i16", "cf32", "cu8"])
def test_threaded_axpy_is_the_same_element_for_element(dtype):
    """The in-place, threaded form (what the CPU baseline times) against the pinned one, over a length
    that is not a multiple of the per-thread chunk and over 3-D shapes."""
    from helpers import make_operand
    for shape in [(3 * 65536 + 77,), (5, 9, 1031), (1,)]:
        for alpha in ([None, (2, 1), (-1, 0)] if oracle.is_complex(dtype) else [None, 3, -1]):
            if alpha is not None and oracle.real_np_dtype(dtype).kind == "u" and (alpha == -1 or alpha == (-1, 0)):
                continue
            x = make_operand(dtype, shape, 51)
            y = make_operand(dtype, shape, 52)
            want = oracle.axpy(dtype, x, alpha, y, contract=True)
            for threads in (1, 3, 0):
                got = y.copy()
                oracle.axpy_inplace(dtype, x, alpha, got, contract=True, threads=threads)
                assert np.array_equal(got, want), f"{dtype} {shape} alpha={alpha} threads={threads}"
