"""CPU: the numpy restatement of random.uniform / transpose / conversions (oracle/tensor_ops.py)
under the reference's own test assertions (src/tensor/random/uniform.zig:215-833), and the host
copy of the hash in the C-ABI library against it."""
import numpy as np
import pytest

from oracle import tensor_ops as ot

REAL = ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64", "f32", "f64"]
ALL = REAL + ["c" + d for d in REAL]


def stats(v):
    v = v.astype(np.float64)
    return v.mean(), v.std()


@pytest.mark.parametrize("dtype", [d for d in ALL if d[-3:] in ("f32", "f64")])
def test_float_without_range_statistics(dtype):
    # uniform.zig:592-648: 10000 values, seed 42, mean 0.5 and stddev 0.289 within 0.05
    v = ot.uniform(dtype, (10000,), 42)
    parts = [v[..., 0], v[..., 1]] if dtype.startswith("c") else [v]
    for p in parts:
        m, s = stats(p)
        assert abs(m - 0.5) < 0.05 and abs(s - 0.289) < 0.05
        assert p.min() >= 0.0 and p.max() <= 1.0


@pytest.mark.parametrize("dtype", REAL[:8])
def test_integer_with_range(dtype):
    # uniform.zig:389-435 and :650-701: values inside [min, max]; mean near the middle
    lo, hi = (0, 100) if dtype[0] == "u" else (-50, 50)
    v = ot.uniform(dtype, (10000,), 42, lo, hi)
    assert v.min() >= lo and v.max() <= hi
    m, s = stats(v)
    assert abs(m - (lo + hi) / 2) < 0.05 * (hi - lo)
    assert abs(s - (hi - lo) / np.sqrt(12)) < 0.05 * (hi - lo)


@pytest.mark.parametrize("dtype", ["f32", "f64", "cf32", "cf64"])
def test_float_with_range(dtype):
    # uniform.zig:437-483 and :764-833
    v = ot.uniform(dtype, (4, 5), 7, -5.0, 5.0)
    assert v.min() >= -5.0 and v.max() <= 5.0 and np.ptp(v) > 1.0


@pytest.mark.parametrize("dtype", REAL[:8])
def test_integer_without_range_uses_the_whole_type(dtype):
    # uniform.zig:703-762: mean near the middle of the type's range
    info = np.iinfo(ot.uniform(dtype, (1,), 0).dtype)
    v = ot.uniform(dtype, (10000,), 42)
    span = float(info.max) - float(info.min)
    assert abs(v.astype(np.float64).mean() - (float(info.max) + float(info.min)) / 2) < 0.05 * span


@pytest.mark.parametrize("dtype", ALL)
def test_seeds(dtype):
    # uniform.zig:485-590: same seed same values, different seeds different values
    a, b, c = ot.uniform(dtype, (3, 4), 100), ot.uniform(dtype, (3, 4), 100), ot.uniform(dtype, (3, 4), 200)
    assert np.array_equal(a, b) and not np.array_equal(a, c)


def test_hash_is_a_bijection_of_the_index_and_avalanches():
    # every step of the hash is invertible in the index, so distinct indices never collide; one flipped
    # input bit flips about half of the output bits
    idx = np.arange(1 << 16, dtype=np.uint64)
    h = ot.hash64(idx, 12345)
    assert len(np.unique(h)) == len(h)
    flips = [bin(int(ot.hash64(np.uint64(1 << b), 9) ^ ot.hash64(np.uint64(0), 9))).count("1") for b in range(64)]
    assert 24 < np.mean(flips) < 40


def test_library_host_hash_matches_the_restatement():
    from wekua_amd import _capi
    lib = _capi.load()
    rng = np.random.default_rng(5)
    for idx, seed in zip(rng.integers(0, 2 ** 63, 200, dtype=np.uint64), rng.integers(0, 2 ** 63, 200, dtype=np.uint64)):
        assert lib.wk_random_hash(int(idx), int(seed)) == int(ot.hash64(idx, int(seed)))
    assert lib.wk_random_hash(0, 0) == int(ot.hash64(np.uint64(0), 0))


def test_transpose_and_conversions_brute_force():
    x = np.arange(2 * 3 * 4).reshape(2, 3, 4)
    t = ot.transpose(x, 0, 2)
    for i in range(2):
        for j in range(3):
            for k in range(4):
                assert t[k, j, i] == x[i, j, k]
    z = np.zeros((2, 2, 2))
    z = ot.to_complex(np.array([[1.0, 2.0], [3.0, 4.0]]), z, 0)
    z = ot.to_complex(np.array([[5.0, 6.0], [7.0, 8.0]]), z, 1)
    assert np.array_equal(z[1, 0], [3.0, 7.0])
    assert np.array_equal(ot.to_real(z, 1), [[5.0, 6.0], [7.0, 8.0]])
