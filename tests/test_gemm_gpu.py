"""GPU parity: wk_gemm (through the C ABI) against the oracle on the same seeded inputs."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import assert_gemm_close, gemm_operands

pytestmark = pytest.mark.gpu

OPS = list(itertools.product((0, 1), (0, 1)))


def run_gemm(dev, dtype, alpha, a, op_a, b, op_b, beta, c, lda=None, ldb=None, ldc=None, packed=False):
    """Uploads dense operands (optionally re-pitched), runs wk_gemm, returns C as dense numpy.
    packed: bring the workspace wk_gemm_workspace_bytes asks for (poisoned first)."""
    cx = oracle.is_complex(dtype)

    def dims(m):
        return m.shape[:2]

    def pitched(m, ld):
        r, cc = dims(m)
        if ld is None or ld == cc:
            return m, cc
        shape = (r, ld) + ((2,) if cx else ())
        out = np.full(shape, 77, dtype=m.dtype)    # poison in the gaps
        out[:, :cc] = m
        return out, ld

    (M, N) = dims(c)
    K = dims(a)[0] if op_a else dims(a)[1]
    ap, lda = pitched(a, lda)
    bp, ldb = pitched(b, ldb)
    cp, ldc = pitched(c, ldc)
    dA, dB, dC = dev.upload(ap), dev.upload(bp), dev.upload(cp)
    ws = None
    if packed:
        from wekua_amd import raw
        need = dev.lib.wk_gemm_workspace_bytes(raw.dtype_id(dtype), op_a, op_b, M, N, K)
        assert need > 0
        ws = dev.upload(np.full(need, 0x5a, dtype=np.uint8))
    dev.gemm(dtype, op_a, op_b, M, N, K, alpha, dA, lda, dB, ldb, beta, dC, ldc, workspace=ws)
    dev.sync()
    out = dC.download(cp.dtype, cp.shape)
    for d in (dA, dB, dC) + ((ws,) if ws is not None else ()):
        d.free()
    if out.shape[1] != N:
        gaps = out[:, N:]
        assert (gaps == 77).all(), "gemm wrote outside the logical region of C"
        out = np.ascontiguousarray(out[:, :N])
    return out


def check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=1, int_range=None, **kw):
    a, b, c = gemm_operands(dtype, M, N, K, op_a, op_b, seed, int_range)
    got = run_gemm(dev, dtype, alpha, a, op_a, b, op_b, beta, c, **kw)
    if M * N * K <= 64 ** 3 * 8:
        want = oracle.semantic_gemm(dtype, alpha, a, op_a, b, op_b, beta, c)
    else:
        want = oracle.gemm(dtype, alpha, a, op_a, b, op_b, beta, c)
    assert_gemm_close(dtype, got, want, alpha, a, op_a, b, op_b, beta, c, K,
                      what=f"{dtype} {M}x{N}x{K} op=({op_a},{op_b}) alpha={alpha} beta={beta}")


SMALL_SHAPES = [(1, 1, 1), (5, 7, 3), (6, 10, 10), (33, 17, 65), (64, 64, 16), (64, 128, 96), (127, 129, 31),
                (130, 70, 200)]


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("op_a,op_b", OPS)
@pytest.mark.parametrize("alpha,beta", [(None, None), (2.0, None), (1.5, 0.5), (None, -0.25)])
def test_float_small_shapes(dev, dtype, op_a, op_b, alpha, beta):
    for (M, N, K) in SMALL_SHAPES:
        check(dev, dtype, M, N, K, op_a, op_b, alpha, beta)


@pytest.mark.parametrize("variant", ["tile64", "mfma_f32_64x64", "mfma_f32_64x64s2", "mfma_f32_64x64s4", "mfma_f32_32x32s4",
                                     "mfma_f32_64x64z", "mfma_f32_128x128", "mfma_f32_128x128s2", "mfma_f32_256x128",
                                     "mfma_f32_128x128t", "mfma_f32_256x128t", "mfma_f32_256x128d", "mfma_f32_128x128d", "mfma_f32_64x64d",
                                     "mfma_f32_128x128d2", "mfma_f32_64x64d2", "mfma_f32_256x128k", "mfma_f32_128x128k", "mfma_f32_64x64k"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_f32_every_variant(dev, variant, op_a, op_b):
    import ctypes
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for (M, N, K) in [(256, 256, 64), (300, 200, 100), (512, 384, 256), (257, 129, 17)]:
            check(dev, "f32", M, N, K, op_a, op_b, 1.5, 0.5, seed=11)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("variant", ["mfma_f32_256x128d", "mfma_f32_128x128d", "mfma_f32_64x64d", "mfma_f64_128x128d", "mfma_f64_64x64d"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_direct_to_lds_with_rows_that_start_anywhere(dev, variant, op_a, op_b):
    """The direct-to-LDS kernels on operands whose rows do not start on 16-byte boundaries (leading dimensions
    that are not multiples of 16 bytes, bases one to three elements into an allocation): four bytes per lane and
    load instead of sixteen.  Several k-slabs with a ragged last one, ragged tiles, poisoned gaps between the rows
    and around the operands, so that a float fetched from the wrong place or a write outside C shows."""
    import ctypes
    from wekua_amd import raw
    dtype = variant[5:8]
    rd = np.float32 if dtype == "f32" else np.float64
    es = np.dtype(rd).itemsize
    poison = rd(7.0e37)
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for (M, N, K), (pa, pb), (sa, sb) in [((300, 200, 100), (1, 3), (1, 2)), ((257, 129, 77), (3, 2), (3, 0)),
                                              ((512, 384, 256), (5, 7), (0, 1)), ((130, 70, 37), (0, 1), (2, 3))]:
            a, b, c = gemm_operands(dtype, M, N, K, op_a, op_b, 91)
            lda, ldb, ldc = a.shape[1] + pa, b.shape[1] + pb, N + 3

            def device_copy(m, ld, shift):
                # rows of ld floats, the whole thing `shift` floats into its allocation, everything else poisoned
                flat = np.full(shift + m.shape[0] * ld + 8, poison, dtype=rd)
                view = flat[shift:shift + m.shape[0] * ld].reshape(m.shape[0], ld)
                view[:, :m.shape[1]] = m
                return dev.upload(flat), flat

            (dA, _), (dB, _), (dC, c_flat) = device_copy(a, lda, sa), device_copy(b, ldb, sb), device_copy(c, ldc, 1)
            ptr = lambda buf, shift: ctypes.c_void_p(buf.ptr.value + es * shift)
            name = dev.lib.wk_gemm_variant(raw.dtype_id(dtype), op_a, op_b, M, N, K, lda, ldb, ldc, ptr(dA, sa), ptr(dB, sb), ptr(dC, 1))
            assert name == variant.encode()
            alpha, beta = raw.scalar_bytes(dtype, 1.5), raw.scalar_bytes(dtype, 0.5)
            raw.check(dev.lib.wk_gemm(dev.stream, raw.dtype_id(dtype), op_a, op_b, M, N, K, ctypes.cast(alpha, ctypes.c_void_p),
                                      ptr(dA, sa), lda, ptr(dB, sb), ldb, ctypes.cast(beta, ctypes.c_void_p), ptr(dC, 1), ldc, None, 0),
                      "wk_gemm")
            dev.sync()
            out = dC.download(rd, c_flat.shape)
            got = out[1:1 + M * ldc].reshape(M, ldc)
            assert (got[:, N:] == poison).all() and out[0] == poison and (out[1 + M * ldc:] == poison).all()
            want = oracle.gemm(dtype, 1.5, a, op_a, b, op_b, 0.5, c)
            assert_gemm_close(dtype, np.ascontiguousarray(got[:, :N]), want, 1.5, a, op_a, b, op_b, 0.5, c, K,
                              what=f"{variant} {M}x{N}x{K} op=({op_a},{op_b}) lda={lda} ldb={ldb} shifts={sa},{sb}")
            for d in (dA, dB, dC):
                d.free()
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("variant", ["tile64", "mfma_f64_64x64", "mfma_f64_64x64s2", "mfma_f64_32x32s4", "mfma_f64_64x64z",
                                     "mfma_f64_128x64", "mfma_f64_128x128", "mfma_f64_128x128d", "mfma_f64_64x64d",
                                     "mfma_f64_128x128k", "mfma_f64_64x64k"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_f64_every_variant(dev, variant, op_a, op_b):
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for (M, N, K) in [(256, 256, 64), (300, 200, 100), (257, 129, 17)]:
            check(dev, "f64", M, N, K, op_a, op_b, 1.0, 1.0, seed=12)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("dtype", ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_integer_wraparound_bit_exact(dev, dtype, op_a, op_b):
    signed = dtype.startswith("i")
    for (M, N, K) in [(5, 7, 3), (33, 17, 65), (64, 128, 96), (130, 70, 200)]:
        for alpha, beta in [(None, None), (3, None), (3, -2 if signed else 250), (None, 7)]:
            check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=21)   # full-range entries: overflow is the norm


@pytest.mark.parametrize("dtype", ["i32", "u32"])
@pytest.mark.parametrize("variant", ["tile64", "mfma_{}_64x128", "mfma_{}_128x128", "mfma_{}_packed"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_int32_every_variant_bit_exact(dev, dtype, variant, op_a, op_b):
    """The int8-matrix-core decomposition (fused and with the pack pass) and the vector-ALU kernel
    against the exact product modulo 2^32 on full-range entries: interior shapes (aligned), ragged
    shapes, K not a multiple of the slab, every alpha / beta combination."""
    variant = variant.format(dtype)
    packed = variant.endswith("packed")
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for (M, N, K) in [(64, 128, 32), (128, 256, 64), (192, 128, 416), (1, 1, 1), (65, 129, 33), (200, 300, 77), (63, 127, 500)]:
            for alpha, beta in [(None, None), (3, None), (-5 if dtype == "i32" else 4000000000, 7), (None, 1)]:
                check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=23, packed=packed)
        if packed:   # unaligned leading dimensions take the element-wise reader of the pack pass
            check(dev, dtype, 130, 70, 200, op_a, op_b, 3, 7, seed=24, packed=True,
                  lda=(130 if op_a else 200) + 3, ldb=(200 if op_b else 70) + 5, ldc=70 + 7)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


def test_int32_packed_needs_its_workspace(dev):
    """Forced packed variant without a workspace (or with one that is too small) is an error, not a
    silent fall-back; with automatic choice a missing workspace just means the fused kernel."""
    from wekua_amd import raw
    a, b, c = gemm_operands("i32", 128, 128, 64, 0, 0, 3)
    dA, dB, dC = dev.upload(a), dev.upload(b), dev.upload(c)
    small = dev.malloc(1024)
    assert dev.lib.wk_gemm_force_variant(b"mfma_i32_packed") == 0
    try:
        lib, p = dev.lib, (dA.ptr, dB.ptr, dC.ptr)
        assert lib.wk_gemm(dev.stream, raw.dtype_id("i32"), 0, 0, 128, 128, 64, None, p[0], 64, p[1], 128, None, p[2], 128, None, 0) == 1
        assert lib.wk_gemm(dev.stream, raw.dtype_id("i32"), 0, 0, 128, 128, 64, None, p[0], 64, p[1], 128, None, p[2], 128, small.ptr, 1024) == 1
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")
    dev.gemm("i32", 0, 0, 128, 128, 64, None, dA, 64, dB, 128, None, dC, 128)
    assert np.array_equal(dC.download(np.int32, (128, 128)), oracle.semantic_gemm("i32", None, a, 0, b, 0, None, c))
    assert dev.lib.wk_gemm_workspace_bytes(raw.dtype_id("f32"), 0, 0, 128, 128, 64) == 0
    for d in (dA, dB, dC, small):
        d.free()


def test_int32_matrix_core_extremes(dev):
    """Inputs built from the byte values that stress the split into balanced signed digits: 0x00, 0x7f,
    0x80, 0xff in every byte position, values whose digits are all -128 or all 127 (every digit pair then
    hits -128 * -128), and values one off a carry into the next digit (0x..7f / 0x..80 at each byte)."""
    import oracle
    vals = np.array([0x00000000, 0x7f7f7f7f, 0x80808080, 0xffffffff, 0x80000000, 0x7fffffff, 0x00800080, 0xff00ff00,
                     0x01010101, 0x807f807f, 0x7f7f7f80, 0x0000007f, 0x00000080, 0x00007f80, 0x007f8000, 0x7f800000,
                     0xffffff80, 0xffffff7f, 0xffff8000, 0x80007fff], dtype=np.uint32)
    M, N, K = 128, 128, 320
    rng = np.random.default_rng(77)
    a = vals[rng.integers(0, len(vals), (M, K))].view(np.int32)
    b = vals[rng.integers(0, len(vals), (K, N))].view(np.int32)
    c = vals[rng.integers(0, len(vals), (M, N))].view(np.int32)
    assert dev.lib.wk_gemm_variant(4, 0, 0, M, N, K, K, N, N, None, None, None).decode().startswith("mfma_i32_")
    dA, dB, dC = dev.upload(a), dev.upload(b), dev.upload(c)
    dev.gemm("i32", 0, 0, M, N, K, -3, dA, K, dB, N, 5, dC, N)
    got = dC.download(np.int32, (M, N))
    want = oracle.semantic_gemm("i32", -3, a, 0, b, 0, 5, c)
    assert np.array_equal(got, want)
    for d in (dA, dB, dC):
        d.free()
    assert dev.lib.wk_gemm_force_variant(b"mfma_i32_packed") == 0
    try:
        assert np.array_equal(run_gemm(dev, "i32", -3, a, 0, b, 0, 5, c, packed=True), want)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


def _fast_exact_i32(alpha, A, B, beta, c):
    """The exact product modulo 2^32 of int32 matrices through float64 products of 16-bit halves (each partial
    product exact below 2^53 for k up to 2^20 or so).  A, B already in op() form."""
    a = A.astype(np.int64)
    b = B.astype(np.int64)
    al, ah = (a & 0xFFFF).astype(np.float64), (a >> 16).astype(np.float64)     # a = ah * 2^16 + al, al unsigned
    bl, bh = (b & 0xFFFF).astype(np.float64), (b >> 16).astype(np.float64)
    ll = (al @ bl).astype(np.uint64)
    mid = ((al @ bh) + (ah @ bl)).astype(np.int64).astype(np.uint64)             # two's complement, then modular
    prod = (ll + (mid << np.uint64(16))) & np.uint64(0xFFFFFFFF)               # ah * bh * 2^32 vanishes
    out = prod
    if alpha is not None or beta is not None:
        out = prod * np.uint64((1 if alpha is None else alpha) & 0xFFFFFFFF)
    if beta is not None:
        out = out + c.astype(np.int64).astype(np.uint64) * np.uint64(beta & 0xFFFFFFFF)
    return (out & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32)


@pytest.mark.parametrize("case", ["small", "two_digits", "big_a_entry", "big_b_entry", "big_a_row", "zero_a", "zero_b",
                                  "minus128", "plus128", "big_in_k_padding_neighbour"])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (1, 1)])
def test_int32_packed_skips_only_empty_digit_planes(dev, case, op_a, op_b):
    """The packed 32-bit product leaves out digit products whose planes the pack pass found all zero, tile by
    tile.  Whatever the magnitudes -- entries of one digit everywhere, of two, one large entry in A only, in B
    only, one large row, an all-zero operand, the values on either side of the first digit's range -- the
    result is the exact product modulo 2^32.  Ragged in every dimension, several tiles, k over several stages."""
    M, N, K = 300, 260, 700
    rng = np.random.default_rng(sum(map(ord, case)))
    lo, hi = (-30000, 30000) if case == "two_digits" else (-100, 100)
    A = rng.integers(lo, hi + 1, (M, K)).astype(np.int32)
    B = rng.integers(lo, hi + 1, (K, N)).astype(np.int32)
    if case == "big_a_entry":
        A[170, 333] = -1234567890
    elif case == "big_b_entry":
        B[650, 259] = 2 ** 31 - 1
    elif case == "big_a_row":
        A[5, :] = rng.integers(-2 ** 31, 2 ** 31, K).astype(np.int32)
    elif case == "zero_a":
        A[:] = 0
    elif case == "zero_b":
        B[:] = 0
    elif case == "minus128":
        A[::7, ::5] = -128         # still one digit
        B[::3, ::11] = -129        # two digits: -129 = 127 - 256
    elif case == "plus128":
        A[::7, ::5] = 127          # one digit
        B[::3, ::11] = 128         # two digits: 128 = -128 + 256
    elif case == "big_in_k_padding_neighbour":
        A[:, K - 1] = 2 ** 24 + 3  # the last real k, next to the zero padding of the planes
        B[K - 1, :] = -(2 ** 24)
    c = rng.integers(-2 ** 31, 2 ** 31, (M, N)).astype(np.int32)
    a = np.ascontiguousarray(A.T) if op_a else A
    b = np.ascontiguousarray(B.T) if op_b else B
    assert dev.lib.wk_gemm_force_variant(b"mfma_i32_packed") == 0
    try:
        for alpha, beta in ((None, None), (3, -2)):
            got = run_gemm(dev, "i32", alpha, a, op_a, b, op_b, beta, c, packed=True)
            want = _fast_exact_i32(alpha, A, B, beta, c)
            bad = np.argwhere(got != want)
            assert len(bad) == 0, f"{case}: {len(bad)} mismatches, first at {bad[0]}"
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


def test_fast_exact_i32_agrees_with_the_semantic_oracle(dev):
    a, b, c = gemm_operands("i32", 40, 30, 50, 0, 0, 9)
    assert np.array_equal(_fast_exact_i32(-7, a, b, 5, c), oracle.semantic_gemm("i32", -7, a, 0, b, 0, 5, c))
    assert np.array_equal(_fast_exact_i32(None, a, b, None, c), oracle.semantic_gemm("i32", None, a, 0, b, 0, None, c))


def _wrapping_u64_product(alpha, A, B, beta, c):
    """alpha * A B + beta * C modulo 2^64 with numpy's wrapping unsigned arithmetic (A, B in op() form)."""
    u = np.uint64
    prod = A.view(u) @ B.view(u) if A.dtype.itemsize == 8 else A.astype(u) @ B.astype(u)
    if alpha is None and beta is None:
        out = prod
    else:
        out = prod * u((1 if alpha is None else alpha) & 0xFFFFFFFFFFFFFFFF)
        if beta is not None:
            out = out + c.view(u) * u(beta & 0xFFFFFFFFFFFFFFFF)
    return out.view(c.dtype)


@pytest.mark.parametrize("dtype", ["i64", "u64"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_int64_packed_bit_exact(dev, dtype, op_a, op_b):
    """64-bit integers on the int8 matrix cores (eight balanced digits, 36 digit products) against the exact
    product modulo 2^64 on full-range entries: interior and ragged shapes, K not a multiple of the k-block,
    every alpha / beta combination, unaligned leading dimensions."""
    variant = f"mfma_{dtype}_packed"
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for (M, N, K) in [(128, 64, 32), (128, 128, 64), (256, 192, 416), (1, 1, 1), (65, 129, 33), (200, 300, 77), (63, 127, 500)]:
            for alpha, beta in [(None, None), (3, None), (-5 if dtype == "i64" else 2 ** 63 + 12345, 7), (None, 1)]:
                check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=31, packed=True)
        check(dev, dtype, 130, 70, 200, op_a, op_b, 3, 7, seed=32, packed=True,
              lda=(130 if op_a else 200) + 3, ldb=(200 if op_b else 70) + 5, ldc=70 + 7)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


def test_int64_packed_digit_extremes_and_long_k(dev):
    """Values that stress the split into eight balanced digits (0x00, 0x7f, 0x80, 0xff in every byte position,
    all digits -128 or all 127, values one off a carry into the next digit), and a k longer than one launch
    may sum exactly (16384): the product is then a chain of launches through C."""
    pieces = np.array([0x00, 0x7f, 0x80, 0xff, 0x01, 0x81, 0x7e, 0xfe], dtype=np.uint64)
    rng = np.random.default_rng(5)

    def draw(shape):
        out = np.zeros(shape, dtype=np.uint64)
        for byte in range(8):
            out |= pieces[rng.integers(0, len(pieces), shape)] << np.uint64(8 * byte)
        return out.view(np.int64)
    tiny_a, tiny_b, tiny_c = draw((9, 40)), draw((40, 7)), draw((9, 7))
    assert np.array_equal(_wrapping_u64_product(-3, tiny_a, tiny_b, 5, tiny_c), oracle.semantic_gemm("i64", -3, tiny_a, 0, tiny_b, 0, 5, tiny_c))
    assert dev.lib.wk_gemm_force_variant(b"mfma_i64_packed") == 0
    try:
        for (M, N, K) in [(128, 64, 320), (130, 70, 16384 + 16384 + 333)]:
            a, b, c = draw((M, K)), draw((K, N)), draw((M, N))
            for alpha, beta in [(None, None), (-3, 5), (7, None)]:
                got = run_gemm(dev, "i64", alpha, a, 0, b, 0, beta, c, packed=True)
                assert np.array_equal(got, _wrapping_u64_product(alpha, a, b, beta, c)), (M, N, K, alpha, beta)
            at, bt = np.ascontiguousarray(a.T), np.ascontiguousarray(b.T)
            got = run_gemm(dev, "i64", 2, at, 1, bt, 1, -1, c, packed=True)
            assert np.array_equal(got, _wrapping_u64_product(2, a, b, -1, c))
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


def test_int64_automatic_choice_with_workspace(dev):
    """With a workspace the automatic choice takes the matrix-core path from mid sizes up and the vector-ALU
    kernel below; both bit-exact, and the name query says which."""
    from wekua_amd import raw
    did = raw.dtype_id("u64")
    name = lambda M, N, K: dev.lib.wk_gemm_variant_with_workspace(did, 0, 0, M, N, K, K, N, N, None, None, None, 1 << 40).decode()
    assert name(512, 512, 512) == "mfma_u64_packed" and name(32, 32, 32) == "tile64"
    for (M, N, K) in [(512, 384, 256), (32, 32, 32)]:
        a, b, c = gemm_operands("u64", M, N, K, 0, 1, 41)
        got = run_gemm(dev, "u64", 3, a, 0, b, 1, 2 ** 64 - 2, c, packed=True)
        assert np.array_equal(got, _wrapping_u64_product(3, a, np.ascontiguousarray(b.T), 2 ** 64 - 2, c))


@pytest.mark.parametrize("op_a,op_b", OPS)
def test_int32_with_workspace_mid_size(dev, op_a, op_b):
    """Mid-size ragged problem with and without a workspace under the automatic choice (which takes
    the packed path only for much larger products) and with the packed path forced: all bit-exact."""
    M, N, K = 768, 896, 300
    a, b, c = gemm_operands("u32", M, N, K, op_a, op_b, 5)
    want = oracle.gemm("u32", 7, a, op_a, b, op_b, 3, c)
    assert np.array_equal(run_gemm(dev, "u32", 7, a, op_a, b, op_b, 3, c, packed=True), want)
    assert np.array_equal(run_gemm(dev, "u32", 7, a, op_a, b, op_b, 3, c), want)
    assert dev.lib.wk_gemm_force_variant(b"mfma_u32_packed") == 0
    try:
        assert np.array_equal(run_gemm(dev, "u32", 7, a, op_a, b, op_b, 3, c, packed=True), want)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("dtype", ["cf32", "cf64", "ci32", "cu16", "ci8", "ci64"])
def test_complex(dev, dtype):
    for op_a, op_b in OPS:
        for (M, N, K) in [(5, 7, 3), (33, 17, 65), (64, 96, 48)]:
            for alpha, beta in [(None, None), ((2, 1), None), ((2, 1), (1, -1))]:
                check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=31)


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32"])
def test_leading_dimensions_and_untouched_gaps(dev, dtype):
    for op_a, op_b in OPS:
        M, N, K = 70, 45, 33
        a_cols = M if op_a else K
        b_cols = K if op_b else N
        check(dev, dtype, M, N, K, op_a, op_b, 2, 3, seed=41, int_range=(-100, 100) if dtype == "i32" else None,
              lda=a_cols + 3, ldb=b_cols + 5, ldc=N + 7)
        check(dev, dtype, M, N, K, op_a, op_b, 2, 3, seed=42, int_range=(-100, 100) if dtype == "i32" else None,
              lda=a_cols + 4, ldb=b_cols + 8, ldc=N + 4)


def test_beta_zero_still_reads_c(dev):
    """gemm.zig:598-602 / gemm_nxn_gpu.cl:280-298: with beta given, C_old is multiplied even if
    beta == 0, so NaN in C propagates; with beta absent C is overwritten."""
    a, b, c = gemm_operands("f32", 64, 64, 64, 0, 0, 5)
    c[:] = np.nan
    out = run_gemm(dev, "f32", 1.0, a, 0, b, 0, 0.0, c)
    assert np.isnan(out).all()
    out = run_gemm(dev, "f32", 1.0, a, 0, b, 0, None, c)
    assert np.isfinite(out).all()


def test_invalid_arguments(dev):
    import ctypes
    from wekua_amd import _capi
    buf = dev.malloc(1024)
    one = ctypes.c_float(1.0)
    lib = dev.lib
    p = buf.ptr
    # zero dimension, bad op, leading dimension too small, bad dtype, null pointer
    assert lib.wk_gemm(dev.stream, 8, 0, 0, 0, 4, 4, None, p, 4, p, 4, None, p, 4, None, 0) == 1
    assert lib.wk_gemm(dev.stream, 8, 2, 0, 4, 4, 4, None, p, 4, p, 4, None, p, 4, None, 0) == 1
    assert lib.wk_gemm(dev.stream, 8, 0, 0, 4, 4, 4, None, p, 3, p, 4, None, p, 4, None, 0) == 1
    assert lib.wk_gemm(dev.stream, 8, 1, 0, 4, 4, 8, None, p, 3, p, 4, None, p, 4, None, 0) == 1
    assert lib.wk_gemm(dev.stream, 8, 0, 0, 4, 4, 4, None, p, 4, p, 4, None, p, 3, None, 0) == 1
    assert lib.wk_gemm(dev.stream, 20, 0, 0, 4, 4, 4, None, p, 4, p, 4, None, p, 4, None, 0) == 9
    assert lib.wk_gemm(dev.stream, 8, 0, 0, 4, 4, 4, None, None, 4, p, 4, None, p, 4, None, 0) == 1
    assert lib.wk_gemm(None, 8, 0, 0, 4, 4, 4, None, p, 4, p, 4, None, p, 4, None, 0) == 1
    # a forced matrix-core variant does not get past the 32-bit limits of its kernel either
    # (automatic selection sends such a problem to the generic kernel); nothing is launched
    for name, dt in ((b"mfma_f32_64x64", 8), (b"mfma_f64_64x64", 9), (b"mfma_i32_64x128", 4)):
        if lib.wk_gemm_force_variant(name) != 0:
            continue
        try:
            assert lib.wk_gemm(dev.stream, dt, 0, 0, 4, 4, 4, None, p, 2 ** 31, p, 4, None, p, 4, None, 0) == 1
            assert lib.wk_gemm(dev.stream, dt, 0, 0, 4, 4, 4, None, p, 4, p, 2 ** 31, None, p, 4, None, 0) == 1
            assert lib.wk_gemm(dev.stream, dt, 0, 0, 4, 4, 4, None, p, 4, p, 4, None, p, 2 ** 31, None, 0) == 1
        finally:
            lib.wk_gemm_force_variant(b"auto")
    buf.free()


@pytest.mark.parametrize("dtype,variant", [("f32", "mfma_f32_64x64"), ("f32", "mfma_f32_64x64s2"), ("f32", "mfma_f32_64x64s4"),
                                           ("f32", "mfma_f32_32x32s4"), ("f32", "mfma_f32_128x128"), ("f32", "mfma_f32_128x128s2"),
                                           ("f32", "mfma_f32_256x128"),
                                           ("f64", "mfma_f64_64x64"), ("f64", "mfma_f64_64x64s2"), ("f64", "mfma_f64_32x32s4"),
                                           ("f64", "mfma_f64_128x64"), ("f64", "mfma_f64_128x128"),
                                           ("f32", "mfma_f32_64x64z"), ("f64", "mfma_f64_64x64z"),
                                           ("f32", "mfma_f32_128x128t"), ("f32", "mfma_f32_256x128t")])
def test_every_k_around_the_slab_boundaries(dev, dtype, variant):
    """Every K from 1 to 100 on a ragged tile and on a tile-aligned shape: the bounds-checked kernels
    choose per-flavour loops from the number of complete slabs (k-slab 16 or 32, one or two slabs of
    prefetch), so every count of slabs from one to a handful, with and without a k tail, must agree."""
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for K in range(1, 101):
            op_a, op_b = K % 2, (K // 2) % 2
            check(dev, dtype, 70, 45, K, op_a, op_b, 1.5, 0.5, seed=100 + K)
            if K % 7 == 0:
                check(dev, dtype, 256, 128, K, op_a, op_b, None, None, seed=300 + K)
                check(dev, dtype, 130, 257, K, 1 - op_a, op_b, 2.0, None, seed=400 + K, lda=(130 if 1 - op_a else K) + 1,
                      ldb=(K if op_b else 257) + 3, ldc=257 + 5)
        for K in (127, 128, 129, 191, 192, 193, 255, 256, 257, 320, 333):    # several slabs of 64 as well
            op_a, op_b = K % 2, (K // 2) % 2
            check(dev, dtype, 70, 45, K, op_a, op_b, 1.5, 0.5, seed=500 + K)
            check(dev, dtype, 128, 192, K, 1 - op_a, op_b, None, None, seed=600 + K)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


def test_one_round_launches_take_the_k_split_tiles(dev):
    """Launches of one round (f32: up to two) of the 64x64 tile with K >= 256 go to its k-split twins;
    the automatic choice is checked by name and its result against the oracle, all four layouts."""
    from wekua_amd import raw

    def name(dtype, M, N, K):
        return dev.lib.wk_gemm_variant(raw.dtype_id(dtype), 0, 0, M, N, K, K, N, N, None, None, None)
    # (the name query assumes 256 compute units and 16-byte aligned operands)
    # f32 operands whose rows start on 16-byte boundaries take the kernels that bring their slabs straight
    # into LDS, whose three stages already give a lone work-group something to overlap with ...
    assert name("f32", 1024, 1024, 1024) == b"mfma_f32_64x64d2"    # one round: two groups of wavefronts per tile
    assert name("f32", 1000, 1000, 1000) == b"mfma_f32_64x64d2"    # ragged, rows of 4000 bytes
    assert name("f32", 2048, 1024, 1024) == b"mfma_f32_64x64d"     # two rounds
    assert name("f32", 1024, 1024, 128) == b"mfma_f32_64x64d"      # short k
    assert name("f32", 1536, 1536, 1536) == b"mfma_f32_64x64k"     # 2.25 tiles per compute unit: two rounds whole, the rest dealt by k-slabs
    assert name("f32", 1408, 1408, 1408) == b"mfma_f32_64x64d"     # 1.89: nearly two whole rounds
    # one full round of 128x128 tiles is between one and two rounds of the 64x64 tile, which then takes its tiles in
    # turn and is the faster one up to k = 2048, except for N,T
    assert name("f32", 2048, 2048, 2048) == b"mfma_f32_64x64d"
    assert name("f32", 2040, 2040, 2040) == b"mfma_f32_64x64d"
    assert name("f32", 2048, 2048, 512) == b"mfma_f32_64x64d"
    assert name("f32", 2048, 2048, 4096) == b"mfma_f32_128x128d2"  # long k: two groups of wavefronts per 128x128 tile
    assert dev.lib.wk_gemm_variant(raw.dtype_id("f32"), 0, 1, 2048, 2048, 2048, 2048, 2048, 2048, None, None, None) == b"mfma_f32_128x128d2"  # N,T
    assert dev.lib.wk_gemm_variant(raw.dtype_id("f32"), 1, 0, 1024, 1024, 1024, 1024, 1024, 1024, None, None, None) == b"mfma_f32_64x64d"  # T,N
    # ... any other leading dimension the same kernels with four bytes per lane and load, one group of wavefronts
    assert name("f32", 1001, 1001, 1001) == b"mfma_f32_64x64d"
    assert name("f32", 2041, 1001, 1001) == b"mfma_f32_64x64d"
    assert name("f32", 1001, 1001, 101) == b"mfma_f32_64x64d"
    assert name("f32", 2042, 2042, 2042) == b"mfma_f32_128x128d"
    assert name("f32", 512, 512, 512) == b"mfma_f32_32x32s4"       # 64 tiles of 64x64 would leave most CUs idle
    assert name("f32", 768, 768, 768) == b"mfma_f32_32x32s4"
    assert name("f64", 1024, 1024, 1024) == b"mfma_f64_64x64d"
    assert name("f64", 1000, 1000, 1000) == b"mfma_f64_64x64d"
    assert name("f64", 1001, 1001, 1001) == b"mfma_f64_64x64d"    # rows of 8008 bytes: four-byte loads
    assert name("f64", 2048, 2048, 2048) == b"mfma_f64_64x64d"
    assert name("f64", 4096, 4096, 4096) == b"mfma_f64_128x128d"
    assert name("f64", 512, 512, 512) == b"mfma_f64_32x32s4"
    for dtype in ("f32", "f64"):
        for op_a, op_b in OPS:
            check(dev, dtype, 1024, 960, 300, op_a, op_b, 1.5, 0.5, seed=93)
            check(dev, dtype, 1000, 1000, 257, op_a, op_b, None, None, seed=94)
            check(dev, dtype, 1001, 999, 257, op_a, op_b, 1.5, 0.5, seed=96)
            check(dev, dtype, 500, 333, 129, op_a, op_b, 2.0, None, seed=95)


@pytest.mark.parametrize("op_a,op_b", OPS)
def test_work_dealt_by_k_slabs(dev, op_a, op_b):
    """Products whose tiles do not fill whole rounds of the compute units have their work dealt by k-slabs
    (mfma_f32_128x128k): tiles are split between work-groups at arbitrary slabs, the parts meet in the stream's
    scratch and are added in the order of k.  The automatic choice by name, every entry against the oracle,
    ragged in every dimension with a k tail, and the same bits on every run (the order of the additions does not
    depend on which work-group arrives last)."""
    from wekua_amd import raw
    M, N, K = 2300, 2500, 2090
    a, b, c = gemm_operands("f32", M, N, K, op_a, op_b, 97)
    up = lambda v: (v + 3) // 4 * 4

    def padded(m):
        out = np.zeros((m.shape[0], up(m.shape[1])), dtype=m.dtype)
        out[:, :m.shape[1]] = m
        return out
    ap, bp, cp = padded(a), padded(b), padded(c)
    lda, ldb, ldc = ap.shape[1], bp.shape[1], cp.shape[1]
    dA, dB = dev.upload(ap), dev.upload(bp)
    name = dev.lib.wk_gemm_variant(raw.dtype_id("f32"), op_a, op_b, M, N, K, lda, ldb, ldc, dA.ptr, dB.ptr, dA.ptr)
    assert name == b"mfma_f32_128x128k"
    want = oracle.gemm("f32", 1.5, a, op_a, b, op_b, 0.5, c, threads=0)
    first = None
    for _ in range(6):
        dC = dev.upload(cp)
        dev.gemm("f32", op_a, op_b, M, N, K, 1.5, dA, lda, dB, ldb, 0.5, dC, ldc)
        dev.sync()
        got = np.ascontiguousarray(dC.download(np.float32, cp.shape)[:, :N])
        dC.free()
        if first is None:
            first = got
            assert_gemm_close("f32", got, want, 1.5, a, op_a, b, op_b, 0.5, c, K, what="work dealt by k-slabs")
        else:
            assert np.array_equal(got, first), "the bits depend on the run"
    # the switch for A/B measurements takes the kernel away
    assert dev.lib.wk_test_option(b"stream_k", 0) == 0
    try:
        assert dev.lib.wk_gemm_variant(raw.dtype_id("f32"), op_a, op_b, M, N, K, lda, ldb, ldc, dA.ptr, dB.ptr, dA.ptr) != b"mfma_f32_128x128k"
    finally:
        dev.lib.wk_test_option(b"stream_k", 1)
    for d in (dA, dB):
        d.free()


@pytest.mark.parametrize("variant,mode,M,N,K,ops", [
    ("mfma_f32_128x128k", 1, 2300, 2500, 700, (0, 0)),    # 360 tiles: 256 run whole, the k-slabs of 104 dealt to 256 work-groups
    ("mfma_f32_128x128k", 2, 2300, 2500, 700, (1, 0)),    # the same product with every tile dealt (768 work-groups)
    ("mfma_f32_256x128k", 1, 4100, 4200, 300, (0, 1)),    # 561 tiles of 256 x 128: two whole rounds, 49 tiles dealt
    ("mfma_f32_256x128k", 1, 2300, 2500, 700, (1, 1)),    # 180 tiles, fewer than compute units: all dealt
    ("mfma_f32_128x128k", 1, 2048, 4096, 520, (0, 0)),    # 512 tiles, whole rounds: the last round dealt one tile each
    ("mfma_f32_128x128k", 1, 1000, 900, 2000, (1, 0)),    # 64 tiles over 768 work-groups: a dozen parts per tile
    ("mfma_f32_256x128k", 2, 4100, 4200, 300, (0, 0)),
    ("mfma_f32_64x64k", 1, 1100, 1300, 1500, (0, 0)),     # 378 tiles of 64 x 64: 256 whole, 122 dealt
    ("mfma_f32_64x64k", 1, 1800, 1700, 600, (1, 0)),      # 783 tiles: three whole rounds (the last starts as slots free up), 15 dealt
    ("mfma_f32_64x64k", 1, 900, 1000, 1100, (0, 1)),      # 240 tiles, fewer than compute units: all dealt
    ("mfma_f32_64x64k", 2, 1100, 1300, 1500, (1, 1)),
    ("mfma_f64_128x128k", 1, 2300, 2500, 360, (0, 0)),    # f64: 360 tiles, 256 whole, 104 dealt
    ("mfma_f64_128x128k", 1, 1000, 900, 1001, (1, 0)),    # 64 tiles over 512 work-groups, a k tail
    ("mfma_f64_128x128k", 2, 2300, 2500, 360, (0, 1)),
    ("mfma_f64_64x64k", 1, 1100, 1300, 750, (1, 1)),      # 378 tiles of 64 x 64
    ("mfma_f64_64x64k", 1, 1800, 1700, 300, (0, 0)),      # 783 tiles: three whole rounds, 15 dealt
    ("mfma_f64_64x64k", 2, 900, 1000, 550, (1, 0))])
def test_work_dealt_by_k_slabs_in_every_form(dev, variant, mode, M, N, K, ops):
    """The kernels that deal k-slabs, forced, in both of their plans (whole rounds of tiles run whole and the rest
    dealt; every tile dealt) and on tile counts below, between and at whole rounds of the compute units: every
    entry against the oracle and the same bits on three runs."""
    op_a, op_b = ops
    dtype = variant[5:8]
    rd = np.float32 if dtype == "f32" else np.float64
    per = 16 // np.dtype(rd).itemsize
    a, b, c = gemm_operands(dtype, M, N, K, op_a, op_b, 131 + mode)
    lda, ldb = a.shape[1], b.shape[1]
    assert lda % per == 0 and ldb % per == 0, "these kernels take rows that start on 16-byte boundaries"
    want = oracle.gemm(dtype, 1.5, a, op_a, b, op_b, 0.5, c, threads=0)
    dA, dB = dev.upload(a), dev.upload(b)
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    assert dev.lib.wk_test_option(b"stream_k", mode) == 0
    try:
        first = None
        for _ in range(3):
            dC = dev.upload(c)
            dev.gemm(dtype, op_a, op_b, M, N, K, 1.5, dA, lda, dB, ldb, 0.5, dC, N)
            dev.sync()
            got = dC.download(rd, c.shape)
            dC.free()
            if first is None:
                first = got
                assert_gemm_close(dtype, got, want, 1.5, a, op_a, b, op_b, 0.5, c, K, what=f"{variant}, plan {mode}")
            else:
                assert np.array_equal(got, first), "the bits depend on the run"
    finally:
        dev.lib.wk_test_option(b"stream_k", 1)
        dev.lib.wk_gemm_force_variant(b"auto")
        dA.free(); dB.free()


@pytest.mark.parametrize("variant,M,N,K,ops", [
    ("mfma_f32_64x64d", 2048, 2048, 96, (1, 0)),      # 1024 tiles on 768 resident work-groups
    ("mfma_f32_64x64d", 1990, 2050, 70, (0, 0)),      # the same count, ragged
    ("mfma_f32_128x128d", 4000, 3900, 48, (0, 1)),    # 992 tiles on 768
    ("mfma_f32_256x128d", 4100, 4200, 40, (1, 1)),    # 561 tiles on 512
    ("mfma_f64_128x128d", 3400, 3400, 40, (0, 0)),    # 729 tiles on 512
    ("mfma_f64_64x64d", 2048, 2000, 36, (1, 0))])     # 1024 tiles on 768
def test_launches_between_one_and_two_rounds_take_their_tiles_in_turn(dev, variant, M, N, K, ops):
    """A launch of more tiles than work-groups are resident at once, but fewer than two rounds of them, is as
    many work-groups as are resident, each taking every n-th tile: every entry against the oracle, and the same
    bits as the launch of one work-group per tile (the test switch)."""
    op_a, op_b = ops
    dtype = variant[5:8]
    rd = np.float32 if dtype == "f32" else np.float64
    a, b, c = gemm_operands(dtype, M, N, K, op_a, op_b, 171)
    want = oracle.gemm(dtype, 1.5, a, op_a, b, op_b, 0.5, c, threads=0)
    dA, dB = dev.upload(a), dev.upload(b)
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        got = {}
        for mode in (1, 0):
            assert dev.lib.wk_test_option(b"persistent", mode) == 0
            dC = dev.upload(c)
            dev.gemm(dtype, op_a, op_b, M, N, K, 1.5, dA, a.shape[1], dB, b.shape[1], 0.5, dC, N)
            dev.sync()
            got[mode] = dC.download(rd, c.shape)
            dC.free()
        assert_gemm_close(dtype, got[1], want, 1.5, a, op_a, b, op_b, 0.5, c, K, what=variant)
        assert np.array_equal(got[0], got[1])
    finally:
        dev.lib.wk_test_option(b"persistent", 1)
        dev.lib.wk_gemm_force_variant(b"auto")
        dA.free(); dB.free()


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_k_split_over_work_groups(dev, dtype):
    """Few tiles of C and a long k: every tile goes to several work-groups, whose partial tiles meet in
    the stream's scratch and are added in a fixed order.  The automatic choice is checked by name and by
    its plan; results against the oracle on all four layouts, aligned and ragged, and twice in a row
    for the same bits (the order of the additions does not depend on which work-group arrives last;
    the arrival counters are back at zero after every launch)."""
    import ctypes
    from wekua_amd import raw
    lib = dev.lib
    did = raw.dtype_id(dtype)
    z = f"mfma_{dtype}_64x64z".encode()
    assert lib.wk_gemm_variant(did, 0, 0, 256, 256, 8192, 8192, 256, 256, None, None, None) == z
    # (64 tiles: in f32 the small tile with all its k-slabs dealt over the resident work-groups measures faster; in
    # f64, whose shares come out even over the units, the split stays)
    assert lib.wk_gemm_variant(did, 0, 0, 512, 512, 8192, 8192, 512, 512, None, None, None) == (b"mfma_f32_64x64k" if dtype == "f32" else z)
    assert lib.wk_gemm_variant(did, 0, 0, 512, 512, 512, 512, 512, 512, None, None, None) != z      # k too short to split
    assert lib.wk_gemm_variant(did, 0, 0, 2048, 2048, 8192, 8192, 2048, 2048, None, None, None) != z  # enough tiles
    shares, klen, first, tiles, nbytes = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_size_t()
    assert lib.wk_gemm_split_plan(did, 0, 0, 512, 512, 8192, z, shares, klen, first, tiles, nbytes) == 0
    # 64 tiles on 256 compute units: shares until four (f32) / two (f64) work-groups sit on every unit
    assert (shares.value, klen.value, tiles.value) == ((16, 512, 64) if dtype == "f32" else (8, 1024, 64))
    for op_a, op_b in OPS:
        check(dev, dtype, 512, 512, 4096, op_a, op_b, 1.5, 0.5, seed=71)           # automatic, aligned
        check(dev, dtype, 300, 200, 4500, op_a, op_b, None, None, seed=72)         # automatic, ragged (k tail in the last share)
        check(dev, dtype, 128, 64, 16500, op_a, op_b, 2.0, None, seed=76)          # two tiles, 64 shares
    assert lib.wk_gemm_force_variant(z) == 0
    try:
        for op_a, op_b in OPS:
            check(dev, dtype, 192, 128, 160, op_a, op_b, 2.0, None, seed=73)       # shares of one or two slabs
            check(dev, dtype, 70, 45, 97, op_a, op_b, 1.5, 0.5, seed=74)           # the last share holds one element of k
            check(dev, dtype, 130, 257, 333, op_a, op_b, None, -0.25, seed=75,
                  lda=(130 if op_a else 333) + 1, ldb=(333 if op_b else 257) + 3, ldc=257 + 5)
        # the same call several times: bit-identical, whoever arrives last
        from helpers import make_operand
        rd = np.float32 if dtype == "f32" else np.float64
        M, N, K = 256, 192, 1024
        a = make_operand(dtype, (M, K), 81)
        b = make_operand(dtype, (K, N), 82)
        dA, dB = dev.upload(a), dev.upload(b)
        outs = []
        for _ in range(4):
            dC = dev.upload(np.zeros((M, N), dtype=rd))
            dev.gemm(dtype, 0, 0, M, N, K, None, dA, K, dB, N, None, dC, N)
            dev.sync()
            outs.append(dC.download(rd, (M, N)))
            dC.free()
        for o in outs[1:]:
            assert np.array_equal(o, outs[0])
        dA.free(); dB.free()
    finally:
        lib.wk_gemm_force_variant(b"auto")
    # The hand-over of partial tiles between work-groups behind different L2s.  Nine tiles: the grid is
    # (tiles, shares) and work-groups go to the eight XCDs in turn by linear number, tile + 9 * share, so
    # the shares of one tile sit on XCDs tile + share (mod 8), eight neighbours on eight different ones.
    # The same launch many times into a poisoned C, every result compared bit for bit with the first and
    # the first with the oracle: a stale partial tile read by the adding work-group would show as a
    # difference.  This is the test to run after a compiler or driver change.
    M = N = 192
    K = 8192
    assert lib.wk_gemm_variant(did, 0, 1, M, N, K, K, K, N, None, None, None) == z
    assert lib.wk_gemm_split_plan(did, 0, 1, M, N, K, None, shares, klen, first, tiles, nbytes) == 0
    assert tiles.value == 9 and shares.value >= 8
    check(dev, dtype, M, N, K, 0, 1, None, None, seed=91)
    a = make_operand(dtype, (M, K), 92)
    b = make_operand(dtype, (N, K), 93)
    dA, dB = dev.upload(a), dev.upload(b)
    dC = dev.upload(np.full((M, N), np.nan, dtype=rd))
    first_bits = None
    for launch in range(24):
        dev.gemm(dtype, 0, 1, M, N, K, None, dA, K, dB, K, None, dC, N)
        dev.sync()
        got = dC.download(rd, (M, N))
        if first_bits is None:
            first_bits = got
        assert np.array_equal(got, first_bits), f"launch {launch} differs from launch 0"
        dC.write(np.full((M, N), np.nan, dtype=rd))
    dA.free(); dB.free(); dC.free()


@pytest.mark.parametrize("variant,bm,bn", [("mfma_f32_256x128d", 256, 128), ("mfma_f32_128x128d", 128, 128), ("mfma_f32_64x64d", 64, 64),
                                           ("mfma_f32_128x128d2", 128, 128), ("mfma_f32_64x64d2", 64, 64),
                                           ("mfma_f64_128x128d", 128, 128), ("mfma_f64_64x64d", 64, 64)])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_slabs_straight_into_lds(dev, variant, bm, bn, op_a, op_b):
    """The kernels that bring their k-slabs from global memory straight into LDS (three stages, swizzled
    layouts): every count of slabs from one to a handful (the pipeline's prologue and its last two
    iterations are special), several tiles, every epilogue, leading dimensions with gaps; against the
    oracle.  Operands whose rows do not start on 16-byte boundaries fall back to the register-staged tile."""
    dtype = variant[5:8]
    per = 4 if dtype == "f32" else 2                 # elements in 16 bytes

    def ragged(M, N, K, alpha, beta, seed):          # rows padded to 16-byte boundaries: these kernels run
        cols_a, cols_b = (M if op_a else K), (K if op_b else N)
        check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=seed,
              lda=-(-cols_a // per) * per, ldb=-(-cols_b // per) * per)
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for K in (16, 32, 48, 64, 80, 96, 112, 128, 256, 1040):
            check(dev, dtype, bm, bn, K, op_a, op_b, 1.5, 0.5, seed=200 + K)
        check(dev, dtype, 2 * bm, 3 * bn, 320, op_a, op_b, None, None, seed=231)
        check(dev, dtype, 3 * bm, 2 * bn, 64, op_a, op_b, 2.0, None, seed=232)
        check(dev, dtype, 9 * bm, 9 * bn, 176, op_a, op_b, None, -0.25, seed=233)          # 81 tiles, more than one group of tile rows
        check(dev, dtype, 2 * bm, 2 * bn, 96, op_a, op_b, 1.5, 0.5, seed=234,
              lda=(2 * bm if op_a else 96) + 8, ldb=(96 if op_b else 2 * bn) + 12, ldc=2 * bn + 5)  # gaps between rows, 16-byte aligned
        check(dev, dtype, 300, 200, 100, op_a, op_b, 1.5, 0.5, seed=235)                  # ragged, dense rows
        # ragged in every dimension: border tiles fetch clamped rows and skip stores, the last slab is
        # zero-filled in LDS beyond K; K below, at and around the slab size, one to three slabs and many
        for K in (1, 3, 4, 15, 17, 31, 33, 47, 50, 100, 1001):
            ragged(bm + 1, 2 * bn - 3, K, 1.5, 0.5, 240 + K)
            check(dev, dtype, bm + 1, 2 * bn - 3, K, op_a, op_b, 1.5, 0.5, seed=240 + K)  # dense rows: whichever kernel takes them
        ragged(2 * bm + 7, bn + 5, 61, None, None, 251)
        ragged(3, 5, 37, 2.0, None, 252)                                                  # smaller than one 16-byte chunk
        ragged(1, 1, 1, 1.5, 0.5, 255)
        ragged(bm - 1, bn - 1, 16, None, -0.25, 253)
        # rows that do not start on 16-byte boundaries: not this kernel's, the staged tile runs
        check(dev, dtype, 2 * bm, bn, 40, op_a, op_b, 1.5, 0.5, seed=254,
              lda=(2 * bm if op_a else 40) + 3, ldb=(40 if op_b else bn) + 1, ldc=bn + 2)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("variant,bm,bn", [("mfma_f32_256x128d", 256, 128), ("mfma_f32_128x128d", 128, 128), ("mfma_f32_64x64d", 64, 64),
                                           ("mfma_f32_64x64d2", 64, 64), ("mfma_f64_128x128d", 128, 128), ("mfma_f64_64x64d", 64, 64)])
def test_tile_walk_in_patches_covers_every_tile_once(dev, variant, bm, bn):
    """The direct-to-LDS kernels number their tiles in XCD-local patches (4 x 8, 4 x 4, 2 x 8 or 2 x 4
    tiles, eight patches at a time) when the tile grid divides into them and in groups of tile rows
    otherwise: one tile grid per patch shape and one that takes none, whole result against the oracle
    (a tile visited twice or not at all leaves entries of C wrong)."""
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for tiles_m, tiles_n in ((8, 32), (8, 16), (2, 64), (2, 32), (16, 16), (6, 10)):
            for op_a, op_b in ((0, 0), (1, 1)):
                check(dev, variant[5:8], tiles_m * bm, tiles_n * bn, 48, op_a, op_b, None, None, seed=300 + tiles_m + tiles_n)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("variant", ["mfma_f32_256x128d", "mfma_f32_128x128d", "mfma_f32_64x64d", "mfma_f32_128x128d2", "mfma_f32_64x64d2",
                                     "mfma_f64_128x128d", "mfma_f64_64x64d"])
def test_direct_to_lds_on_seeded_random_shapes(dev, variant):
    """Twenty-four shapes drawn from a fixed seed (1 <= M, N <= 700, 1 <= K <= 900), rows of 16-byte multiples
    with or without a gap, every layout and option combination in turn: the kernels that bring their slabs
    straight into LDS against the oracle, border tiles and k tails included."""
    rng = np.random.default_rng(20240611)
    dtype = variant[5:8]
    per = 4 if dtype == "f32" else 2
    options = [(None, None), (2.0, None), (1.5, 0.5), (None, -0.25)]
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for n in range(24):
            M, N, K = int(rng.integers(1, 701)), int(rng.integers(1, 701)), int(rng.integers(1, 901))
            op_a, op_b = OPS[n % 4]
            alpha, beta = options[(n // 4) % 4]
            cols_a, cols_b = (M if op_a else K), (K if op_b else N)
            pad = per * int(rng.integers(0, 3))
            check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=400 + n,
                  lda=-(-cols_a // per) * per + pad, ldb=-(-cols_b // per) * per + pad, ldc=N + int(rng.integers(0, 4)))
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("dtype,M,N,K,split", [("f32", 4097, 4095, 1024, True),    # one row beyond sixteen tiles of 256
                                                ("f32", 2050, 4097, 1536, True),    # two rows and one column beyond
                                                ("f32", 4096, 4100, 1024, True),    # four columns beyond
                                                ("f32", 4097, 4095, 64, False),     # short k: a launch more costs more than it saves
                                                ("f32", 4160, 4096, 1024, True),    # 64 rows beyond: a quarter of the tile, still thin
                                                ("f32", 4225, 4096, 1024, True),    # one row beyond 33 tiles of 128
                                                ("f32", 4200, 4096, 1024, True),    # 104 rows beyond: split off because the cost model says so
                                                ("f32", 3000, 3000, 1024, False),   # ... and here it does not: the body would fill half a round
                                                ("f32", 2049, 2047, 1024, False),   # the body is too small to carry a strip's launch
                                                ("f64", 3073, 3072, 1024, True),    # f64: one row beyond 24 tiles of 128
                                                ("f64", 2049, 2050, 1024, False)])  # the whole, with its left-over tiles dealt by k-slabs, is cheaper
def test_thin_strips_beyond_whole_tiles_are_products_of_their_own(dev, dtype, M, N, K, split):
    """A matrix a few rows or columns larger than whole large tiles is multiplied in parts (the body of whole
    tiles, then the thin strips beyond it, each with its own kernel) when k is long and the body large enough
    to carry the extra launches; the name query marks it.  Every entry of C against the oracle, all four layouts, rows of 16-byte
    multiples (which is what tensors have), C with a gap between rows whose poison must survive."""
    from wekua_amd import raw
    per = 4 if dtype == "f32" else 2
    up = lambda n: -(-n // per) * per
    for op_a, op_b in OPS:
        lda, ldb = up(M if op_a else K), up(K if op_b else N)
        name = dev.lib.wk_gemm_variant(raw.dtype_id(dtype), op_a, op_b, M, N, K, lda, ldb, N + 3, None, None, None).decode()
        assert name.endswith("+strips") == split, (name, op_a, op_b)
        check(dev, dtype, M, N, K, op_a, op_b, 1.5, 0.5, seed=500 + op_a * 2 + op_b, lda=lda, ldb=ldb, ldc=N + 3)
    check(dev, dtype, M, N, K, 0, 1, None, None, seed=505, lda=up(K), ldb=up(K))


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_thin_products(dev, dtype, op_a, op_b):
    """At most four rows or four columns of C (matrix-vector products in all but name): the kernels that read
    the long operand once along its storage order, one to four rows / columns, k below, at and beyond the
    1024 values of the thin operand that LDS holds at a time, every epilogue, rows of 16-byte multiples and
    not (the vector and the scalar loads), gaps between the rows of C whose poison must survive; against the
    oracle.  The name query says which products take them."""
    from wekua_amd import raw
    per = 4 if dtype == "f32" else 2
    up = lambda n: -(-n // per) * per
    did = raw.dtype_id(dtype)

    def name(M, N, K):
        return dev.lib.wk_gemm_variant(did, op_a, op_b, M, N, K, M if op_a else K, K if op_b else N, N, None, None, None)
    assert name(1, 4095, 4093) == b"thin" and name(4096, 1, 4093) == b"thin" and name(4, 512, 128) == b"thin"
    assert name(5, 4095, 4093) != b"thin" and name(1, 500, 4093) != b"thin" and name(2, 3, 4093) != b"thin" and name(1, 4095, 100) != b"thin"
    options = [(None, None), (2.0, None), (1.5, 0.5), (None, -0.25)]
    n = 0
    for (M, N, K) in [(1, 4095, 4093), (4096, 1, 4093), (3, 1000, 700), (700, 4, 1024), (2, 513, 129), (1031, 2, 2050),
                      (4, 2048, 1025), (600, 3, 128)]:
        alpha, beta = options[n % 4]
        cols_a, cols_b = (M if op_a else K), (K if op_b else N)
        check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=600 + n)                                   # dense rows
        check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=620 + n, lda=up(cols_a) + per, ldb=up(cols_b), ldc=N + 3)
        n += 1


SKINNY_SHAPES = [(32, 4096, 2048), (17, 4100, 1100), (5, 8190, 600), (16, 3001, 1500), (9, 4096, 1030), (31, 260, 17000), (2, 4096, 2048),
                 (4096, 32, 2048), (4100, 9, 1100), (8190, 24, 777), (3001, 16, 1500), (300, 7, 16001), (4099, 3, 1100), (4, 8190, 600),
                 (17, 2100, 2090), (2100, 24, 2053), (64, 4096, 2048), (33, 4100, 2100), (4100, 48, 2090), (8190, 64, 600)]


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_skinny_products(dev, dtype, op_a, op_b):
    """Five to 32 rows or columns of C against a large other operand (a small batch through a weight matrix):
    the kernel that streams the large operand once into registers.  One and two blocks of sixteen on the short
    side, both storage orders of both operands, k with every kind of tail (a last group of k that is partial, a
    last share that is short), ragged long sides, every epilogue, gaps between the rows of all three matrices
    whose poison must survive; against the oracle.  The name query says which products take it, and the test
    option takes it away."""
    from wekua_amd import raw
    per = 4 if dtype == "f32" else 2
    up = lambda n: -(-n // per) * per
    did = raw.dtype_id(dtype)

    def name(M, N, K, lda=None, ldb=None):
        return dev.lib.wk_gemm_variant(did, op_a, op_b, M, N, K, lda or up(M if op_a else K), ldb or up(K if op_b else N), N, None, None, None)
    assert name(32, 4096, 2048) == b"skinny" and name(4096, 32, 2048) == b"skinny" and name(5, 8192, 512) == b"skinny"
    assert name(65, 4096, 2048) != b"skinny" and name(32, 1024, 1024) != b"skinny"
    # one row or column stays with the thin kernel (a matrix-vector product); two to four come here where the long
    # operand is large and its rows start on 16-byte boundaries
    assert name(1, 4096, 2048) == b"thin" and name(4, 4096, 2048) == b"skinny" and name(4096, 2, 2048) == b"skinny" and name(4, 512, 128) == b"thin"
    assert name(32, 32, 1 << 20) != b"skinny" and name(32, 1 << 20, 128) != b"skinny"
    # a leading dimension of the large operand that is no multiple of 16 bytes: the tile kernels' business
    assert name(32, 4095, 2047, ldb=2047 if op_b else 4095) != b"skinny"
    assert dev.lib.wk_test_option(b"skinny", 0) == 0
    try:
        assert name(32, 4096, 2048) != b"skinny"
    finally:
        dev.lib.wk_test_option(b"skinny", 1)
    options = [(1.5, 0.5), (None, None), (2.0, None), (None, -0.25)]
    for n, (M, N, K) in enumerate(SKINNY_SHAPES):
        alpha, beta = options[n % 4]
        cols_a, cols_b = (M if op_a else K), (K if op_b else N)
        # (f32 with more than sixteen on the short side and k below 2048 stays with the tile kernels, which start
        # faster; 33 to 64 on the short side come here with a large operand that is contiguous along the long side,
        # in f32 only with a short operand that allows 16-byte loads along k)
        expect = not (dtype == "f32" and min(M, N) > 16 and K < 2048)
        if min(M, N) > 32:
            big_k, s_kc = (op_b != 0, op_a == 0) if M <= N else (op_a == 0, op_b != 0)
            expect = expect and not big_k and (s_kc or dtype == "f64")
        assert (name(M, N, K) == b"skinny") == expect, (M, N, K)
        check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=700 + n, lda=up(cols_a), ldb=up(cols_b), ldc=N)
        check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=720 + n, lda=up(cols_a) + per, ldb=up(cols_b) + 2 * per, ldc=N + 3)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_skinny_products_give_the_same_bits_on_every_run(dev, dtype):
    """k is split over the wavefronts of a work-group and over work-groups; the sums are added in the order of
    k whichever work-group arrives last.  Also with two to four work-groups per unit instead of the default
    (other shares of k, so other bits between the settings, the same within one)."""
    rd = np.float32 if dtype == "f32" else np.float64
    for (M, N, K, op_a, op_b) in [(32, 4096, 8192, 0, 0), (8192, 12, 4096, 0, 1), (20, 8192, 4096, 1, 1)]:
        a, b, c = gemm_operands(dtype, M, N, K, op_a, op_b, 333)
        want = oracle.gemm(dtype, 1.5, a, op_a, b, op_b, 0.5, c, threads=0)
        dA, dB = dev.upload(a), dev.upload(b)
        for per_unit in (1, 2, 4):
            assert dev.lib.wk_test_option(b"skinny", per_unit) == 0
            try:
                first = None
                for _ in range(4):
                    dC = dev.upload(c)
                    dev.gemm(dtype, op_a, op_b, M, N, K, 1.5, dA, a.shape[1], dB, b.shape[1], 0.5, dC, N)
                    dev.sync()
                    got = dC.download(rd, c.shape)
                    dC.free()
                    if first is None:
                        first = got
                        assert_gemm_close(dtype, got, want, 1.5, a, op_a, b, op_b, 0.5, c, K, what=f"skinny {M}x{N}x{K}, {per_unit} per unit")
                    else:
                        assert np.array_equal(got, first), "the bits depend on the run"
            finally:
                dev.lib.wk_test_option(b"skinny", 1)
        dA.free(); dB.free()


def test_left_over_tiles_run_as_a_k_split_tail(dev):
    """A launch whose tiles do not fill whole rounds of the compute units: the whole rounds run as they
    are, the left-over tiles as a second launch with k split over work-groups.  Checked: the plan of the
    automatic choice for the ragged benchmark shape, results against the oracle for body + tail (forced
    on shapes of a few hundred tiles, all layouts, aligned and ragged), and the same bits on every run."""
    import ctypes
    from helpers import make_operand
    from wekua_amd import raw
    lib = dev.lib
    did = raw.dtype_id("f32")
    shares, klen, first, tiles, nbytes = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_size_t()
    # 4097 x 4095 in tiles of 256 x 128: 17 x 32 = 544 = two rounds of 256 and 32 left over
    assert lib.wk_gemm_split_plan(did, 0, 0, 4097, 4095, 4093, b"mfma_f32_256x128t", shares, klen, first, tiles, nbytes) == 0
    assert (first.value, tiles.value) == (512, 32) and shares.value >= 2 and klen.value % 16 == 0
    assert nbytes.value == shares.value * 32 * 256 * 128 * 4 <= 64 << 20
    # a product of whole rounds has no tail; the variant then runs the plain tile
    assert lib.wk_gemm_split_plan(did, 0, 0, 4096, 4096, 4096, b"mfma_f32_256x128t", shares, klen, first, tiles, nbytes) == 0
    assert shares.value == 1
    for variant, (M, N) in ((b"mfma_f32_128x128t", (2100, 2000)), (b"mfma_f32_256x128t", (4097, 2047))):
        assert lib.wk_gemm_force_variant(variant) == 0
        try:
            for op_a, op_b in OPS:
                check(dev, "f32", M, N, 160, op_a, op_b, 1.5, 0.5, seed=83)         # 272 tiles: one round + 16
                check(dev, "f32", M, N - 5, 67, op_a, op_b, None, None, seed=84)    # k tail inside the last share
            check(dev, "f32", 300, 200, 100, 0, 1, 2.0, None, seed=85)              # less than a round: all tail
            a = make_operand("f32", (2100, 192), 86)
            b = make_operand("f32", (192, 2000), 87)
            dA, dB = dev.upload(a), dev.upload(b)
            outs = []
            for _ in range(3):
                dC = dev.upload(np.zeros((2100, 2000), dtype=np.float32))
                dev.gemm("f32", 0, 0, 2100, 2000, 192, None, dA, 192, dB, 2000, None, dC, 2000)
                dev.sync()
                outs.append(dC.download(np.float32, (2100, 2000)))
                dC.free()
            assert np.array_equal(outs[1], outs[0]) and np.array_equal(outs[2], outs[0])
            dA.free(); dB.free()
        finally:
            lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("variant", ["mfma_i32_64x128", "mfma_i32_128x128", "mfma_i32_packed"])
def test_int32_every_k(dev, variant):
    """K from 1 to 70 (one to three k-slabs, every tail length; for the pack pass also fewer k-blocks
    than k-ranges of its grid) on a ragged shape, full-range entries, bit-exact."""
    packed = variant.endswith("packed")
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        for K in range(1, 71):
            op_a, op_b = K % 2, (K // 2) % 2
            check(dev, "i32", 70, 130, K, op_a, op_b, -7, 3, seed=500 + K, packed=packed)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("dtype", ["i8", "u8", "i16", "u16"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_narrow_integers_packed_bit_exact(dev, dtype, op_a, op_b):
    """8- and 16-bit integers on the int8 matrix cores (pack pass + packed kernel with one or two digits
    per element) against the exact product modulo 2^8 / 2^16: full-range entries, aligned and ragged
    shapes, K around the slab boundaries (a slab is 128 / 64 values of k), odd leading dimensions."""
    signed = dtype.startswith("i")
    assert dev.lib.wk_gemm_force_variant(f"mfma_{dtype}_packed".encode()) == 0
    try:
        for (M, N, K) in [(128, 128, 128), (256, 128, 64), (1, 1, 1), (65, 129, 33), (200, 300, 77), (63, 127, 500), (130, 70, 129)]:
            for alpha, beta in [(None, None), (3, None), (-5 if signed else 201, 7), (None, 1)]:
                check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=61, packed=True)
        for K in (31, 32, 63, 64, 65, 127, 128, 191, 192, 257):
            check(dev, dtype, 70, 45, K, op_a, op_b, 3, 2, seed=62 + K, packed=True)
        check(dev, dtype, 130, 70, 200, op_a, op_b, 3, 7, seed=64, packed=True,
              lda=(130 if op_a else 200) + 3, ldb=(200 if op_b else 70) + 5, ldc=70 + 7)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("dtype", ["u8", "i16"])
def test_narrow_integers_packed_large_tile(dev, dtype):
    """From one 256 x 128 tile per compute unit up the packed kernel runs that tile (64 x 64 per
    wavefront): an aligned and a ragged problem of that many tiles with a short K, bit-exact."""
    assert dev.lib.wk_gemm_force_variant(f"mfma_{dtype}_packed".encode()) == 0
    try:
        check(dev, dtype, 4096, 2048, 128, 0, 1, None, None, seed=65, packed=True)
        check(dev, dtype, 4096 + 77, 2048 + 5, 96, 1, 0, 3, 7, seed=66, packed=True)
        if dtype == "i16":  # (its pipeline runs stages of 32 k, a multiple of four of them: twelve and twenty here)
            check(dev, dtype, 4096, 2048, 300, 0, 0, 3, None, seed=71, packed=True)
            check(dev, dtype, 4096 + 1, 2048 + 127, 520, 1, 1, None, -2, seed=72, packed=True)
        if dtype == "u8":   # and from one 256 x 256 tile per compute unit up the 8-bit types run that one
            check(dev, dtype, 4096, 4096, 128, 0, 1, None, 5, seed=67, packed=True)
            check(dev, dtype, 4096 + 77, 4096 + 5, 96, 1, 0, 3, 7, seed=68, packed=True)
            # (its pipeline runs stages of 64 k, a multiple of four of them: four, eight and twelve here)
            check(dev, dtype, 4096, 4096, 300, 0, 0, 3, None, seed=69, packed=True)
            check(dev, dtype, 4096 + 1, 4096 + 255, 520, 1, 1, None, None, seed=70, packed=True)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("dtype", ["i8", "u16"])
def test_narrow_integers_with_workspace_automatic(dev, dtype):
    """With a workspace the automatic choice takes the matrix cores from a few hundred cubed up; the
    result equals the vector-ALU kernel's (no workspace) and the oracle's."""
    M, N, K = 768, 640, 1024
    a, b, c = gemm_operands(dtype, M, N, K, 0, 1, 7)
    from wekua_amd import raw
    need = dev.lib.wk_gemm_workspace_bytes(raw.dtype_id(dtype), 0, 1, M, N, K)
    assert dev.lib.wk_gemm_variant_with_workspace(raw.dtype_id(dtype), 0, 1, M, N, K, K, K, N, None, None, None, need) \
        == f"mfma_{dtype}_packed".encode()
    want = oracle.gemm(dtype, 3, a, 0, b, 1, 5, c)
    assert np.array_equal(run_gemm(dev, dtype, 3, a, 0, b, 1, 5, c, packed=True), want)
    assert np.array_equal(run_gemm(dev, dtype, 3, a, 0, b, 1, 5, c), want)


def test_complex_integers_with_workspace_automatic(dev):
    """ci16 at a size where the automatic choice takes the pack passes: same bits as the generic
    kernel (no workspace) and the oracle."""
    from wekua_amd import raw
    dtype, (M, N, K) = "ci16", (512, 384, 512)
    a, b, c = gemm_operands(dtype, M, N, K, 1, 0, 9)
    need = dev.lib.wk_gemm_workspace_bytes(raw.dtype_id(dtype), 1, 0, M, N, K)
    assert dev.lib.wk_gemm_variant_with_workspace(raw.dtype_id(dtype), 1, 0, M, N, K, M, N, N, None, None, None, need) \
        == b"mfma_ci16_packed"
    want = oracle.gemm(dtype, (3, -2), a, 1, b, 0, (5, 1), c)
    assert np.array_equal(run_gemm(dev, dtype, (3, -2), a, 1, b, 0, (5, 1), c, packed=True), want)
    assert np.array_equal(run_gemm(dev, dtype, (3, -2), a, 1, b, 0, (5, 1), c), want)
    # cu32 at a size below its own pack pass: the real product runs on the fused int8 matrix-core kernel
    for (M, N, K, op_a, op_b) in [(256, 192, 320, 0, 1), (130, 70, 200, 1, 1)]:
        a, b, c = gemm_operands("cu32", M, N, K, op_a, op_b, 10)
        want = oracle.gemm("cu32", (4000000000, 7), a, op_a, b, op_b, (1, 2), c)
        assert np.array_equal(run_gemm(dev, "cu32", (4000000000, 7), a, op_a, b, op_b, (1, 2), c, packed=True), want)


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u8", "i16"])
def test_seeded_random_problems(dev, dtype):
    """Sixty seeded random problems per type under the automatic kernel choice: shapes up to 400 (so
    that every tile of the cost model and both bounds-checked flavours come up), random transposes,
    option combinations and leading-dimension padding; the integer types also with a workspace."""
    rng = np.random.default_rng({"f32": 1, "f64": 2, "i32": 3, "u8": 4, "i16": 5}[dtype])
    integer = dtype[0] in "iu"
    for case in range(60):
        M, N, K = (int(v) for v in rng.integers(1, 401, 3))
        if case % 5 == 0:
            M, N, K = (M + 63) // 64 * 64, (N + 63) // 64 * 64, (K + 31) // 32 * 32    # tile-aligned: the unchecked kernels
        op_a, op_b = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        mode = int(rng.integers(0, 4))
        if integer:
            alpha, beta = [(None, None), (3, None), (5, 7), (None, 1)][mode]
        else:
            alpha, beta = [(None, None), (2.0, None), (1.5, 0.5), (None, -0.25)][mode]
        pad = int(rng.integers(0, 3)) * int(rng.integers(1, 9))
        a_cols, b_cols = (M if op_a else K), (K if op_b else N)
        kw = dict(lda=a_cols + pad, ldb=b_cols + pad, ldc=N + pad) if pad else {}
        check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=1000 + case, packed=integer and case % 2 == 0, **kw)


@pytest.mark.parametrize("dtype", ["cf32", "cf64", "ci8", "cu8", "ci16", "cu16", "ci32", "cu32", "ci64", "cu64"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_complex_through_the_real_matrix_cores(dev, dtype, op_a, op_b):
    """Complex types with a workspace: B is expanded to its real 2K x 2N form (alpha folded in),
    transposed operands are turned first, beta scales C beforehand, and the product is the real
    matrix-core path on (M, 2N, 2K) -- the f32 / f64 kernel, or for the complex integers the packed
    int8 matrix-core path, where every step is exact modulo 2^width.  Against the oracle (floats to
    the tolerance of the real types, integers bit for bit on full-range entries), for every option
    combination, ragged shapes and padded leading dimensions."""
    assert dev.lib.wk_gemm_force_variant(f"mfma_{dtype}_packed".encode()) == 0
    fl = dtype[1] == "f"
    try:
        for (M, N, K) in [(5, 7, 3), (33, 17, 65), (64, 96, 48), (128, 128, 64), (130, 70, 200), (257, 129, 17)]:
            for alpha, beta in [(None, None), ((2, 1), None), ((2, 1), (1, -1)), (None, (0.5, 0.25) if fl else (3, 125))]:
                check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=71, packed=True)
        check(dev, dtype, 70, 45, 33, op_a, op_b, (1.5, -0.5) if fl else (-7, 5), (0.25, 2) if fl else (2, -3), seed=72, packed=True,
              lda=(70 if op_a else 33) + 3, ldb=(33 if op_b else 45) + 5, ldc=45 + 7)
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


def test_complex_float_nan_in_c_propagates_with_beta(dev):
    """beta given: C_old is read and multiplied (so NaN propagates) also on the packed path."""
    a, b, c = gemm_operands("cf32", 64, 64, 64, 0, 0, 5)
    c[:] = np.nan
    assert dev.lib.wk_gemm_force_variant(b"mfma_cf32_packed") == 0
    try:
        assert np.isnan(run_gemm(dev, "cf32", (1, 0), a, 0, b, 0, (0, 0), c, packed=True)).all()
        assert np.isfinite(run_gemm(dev, "cf32", (1, 0), a, 0, b, 0, None, c, packed=True)).all()
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("dtype", ["i8", "u16", "i32", "u64", "cf32", "cf64", "ci16", "cu32", "ci64"])
@pytest.mark.parametrize("op_a,op_b", OPS)
def test_packed_b_kept_across_calls(dev, dtype, op_a, op_b):
    """wk_gemm_packed_b_kept: after one wk_gemm with a workspace, later calls with a new A pack only A.
    To show that B's packed form in the workspace is what the product reads, B's own buffer is
    overwritten with other values before the second call: the result must still be the product
    with the first B.  A third, ordinary wk_gemm then sees the new B."""
    from wekua_amd import raw
    forced = f"mfma_{dtype}_packed".encode()
    assert dev.lib.wk_gemm_force_variant(forced) == 0
    try:
        for (M, N, K), alpha, beta in [((128, 128, 64), None, None), ((130, 70, 200), (2, 1) if dtype.startswith("c") else 3, None),
                                       ((65, 129, 33), (1.5, -0.5) if dtype.startswith("c") else 2,
                                        (0.25, 2) if dtype.startswith("c") else 5)]:
            a1, b1, c0 = gemm_operands(dtype, M, N, K, op_a, op_b, 81)
            a2, b2, _ = gemm_operands(dtype, M, N, K, op_a, op_b, 82)
            dA, dB, dC = dev.upload(a1), dev.upload(b1), dev.upload(c0)
            need = dev.lib.wk_gemm_workspace_bytes(raw.dtype_id(dtype), op_a, op_b, M, N, K)
            ws = dev.upload(np.full(need, 0x5a, dtype=np.uint8))
            lda, ldb = a1.shape[1], b1.shape[1]

            def product(a, b, b_kept):
                dC.write(c0)
                dev.gemm(dtype, op_a, op_b, M, N, K, alpha, dA, lda, dB, ldb, beta, dC, N, workspace=ws, b_kept=b_kept)
                dev.sync()
                got = dC.download(c0.dtype, c0.shape)
                want = oracle.gemm(dtype, alpha, a, op_a, b, op_b, beta, c0)
                assert_gemm_close(dtype, got, want, alpha, a, op_a, b, op_b, beta, c0, K,
                                  what=f"{dtype} {M}x{N}x{K} op=({op_a},{op_b}) b_kept={b_kept}")

            product(a1, b1, False)
            dA.write(a2)
            dB.write(b2)                    # B's buffer changes; its packed form in the workspace does not
            product(a2, b1, True)
            dA.write(a1)
            product(a1, b1, True)           # and again, A back to the first
            product(a1, b2, False)          # an ordinary call packs the new B
            dA.write(a2)
            product(a2, b2, True)
            for d in (dA, dB, dC, ws):
                d.free()
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


def test_packed_b_kept_is_plain_gemm_without_a_workspace_path(dev):
    """Types and sizes that do not use the workspace: the entry point is wk_gemm."""
    for dtype, (M, N, K) in [("f32", (130, 70, 200)), ("i64", (33, 17, 65)), ("i32", (64, 64, 64))]:
        a, b, c = gemm_operands(dtype, M, N, K, 0, 1, 83)
        dA, dB, dC = dev.upload(a), dev.upload(b), dev.upload(c)
        dev.gemm(dtype, 0, 1, M, N, K, None, dA, K, dB, K, None, dC, N, b_kept=True)
        dev.sync()
        got = dC.download(c.dtype, c.shape)
        want = oracle.semantic_gemm(dtype, None, a, 0, b, 1, None, c)
        assert_gemm_close(dtype, got, want, None, a, 0, b, 1, None, c, K, what=dtype)
        for d in (dA, dB, dC):
            d.free()


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_seeded_random_mid_size_problems(dev, dtype):
    """Sixteen seeded random problems per type with M, N up to 2300 and K up to 700 under the automatic
    kernel choice: the sizes where it moves between the quarter-size tile, the k-split twins, the plain
    64x64 tile and the 128x128 tiles, mostly through their bounds-checked instantiations."""
    from wekua_amd import raw
    rng = np.random.default_rng({"f32": 11, "f64": 12}[dtype])
    seen = set()
    for case in range(16):
        M, N = (int(v) for v in rng.integers(300, 2301, 2))
        K = int(rng.integers(64, 701))
        if case % 4 == 0:
            M, N, K = (M + 127) // 128 * 128, (N + 127) // 128 * 128, (K + 63) // 64 * 64   # the unchecked kernels
        op_a, op_b = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        alpha, beta = [(None, None), (1.5, None), (1.5, 0.5), (None, -0.25)][case % 4]
        seen.add(dev.lib.wk_gemm_variant(raw.dtype_id(dtype), op_a, op_b, M, N, K, M if op_a else K, K if op_b else N, N, None, None,
                                         None))
        check(dev, dtype, M, N, K, op_a, op_b, alpha, beta, seed=700 + case)
    assert len(seen) >= 2, seen
