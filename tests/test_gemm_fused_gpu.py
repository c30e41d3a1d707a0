"""GPU: wk_gemm_bias_activation (one matrix of Linear.forward, src/nn/layer/linear.zig:480-525) against
the two calls it replaces, wk_gemm followed by wk_bias_activation, to the bit, and against the oracle
(oracle/nn.py linear forward) to the activation's tolerance."""
import ctypes

import numpy as np
import pytest

import oracle
from oracle import nn as onn
from wekua_amd import raw

pytestmark = pytest.mark.gpu
ACT = {"none": -1, "sigmoid": 0, "tanh": 1}


def both(dev, dtype, M, N, K, op_a, op_b, kind, with_bias, seed, ld_extra=0):
    rd = oracle.real_np_dtype(dtype)
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1, 1, ((K, M) if op_a else (M, K))).astype(rd)
    b = rng.uniform(-1, 1, ((N, K) if op_b else (K, N))).astype(rd)
    bias = rng.uniform(-1, 1, N).astype(rd)
    lda, ldb, ldc = a.shape[1] + ld_extra, b.shape[1] + ld_extra, N + ld_extra

    def padded(m, ld):
        out = np.full((m.shape[0], ld), 7, dtype=rd)
        out[:, :m.shape[1]] = m
        return out
    dA, dB, dbias = dev.upload(padded(a, lda)), dev.upload(padded(b, ldb)), dev.upload(bias)
    c0 = np.full((M, ldc), 5, dtype=rd)
    d1, d2 = dev.upload(c0), dev.upload(c0)
    bp = dbias.ptr if with_bias else None
    lib, did = dev.lib, raw.dtype_id(dtype)
    raw.check(lib.wk_gemm_bias_activation(dev.stream, did, op_a, op_b, M, N, K, dA.ptr, lda, dB.ptr, ldb, d1.ptr, ldc, bp, ACT[kind]),
              "fused")
    dev.gemm(dtype, op_a, op_b, M, N, K, None, dA, lda, dB, ldb, None, d2, ldc)
    raw.check(lib.wk_bias_activation(dev.stream, did, ACT[kind], M, N, d2.ptr, ldc, bp), "bias_activation")
    dev.sync()
    fused, two = d1.download(rd, (M, ldc)), d2.download(rd, (M, ldc))
    for d in (dA, dB, dbias, d1, d2):
        d.free()
    assert (fused[:, N:] == 5).all() and (two[:, N:] == 5).all()
    A = a.T if op_a else a
    B = b.T if op_b else b
    return fused[:, :N], two[:, :N], A, B, bias if with_bias else None


@pytest.mark.parametrize("dtype,variant", [("f32", "auto"), ("f32", "mfma_f32_64x64"), ("f32", "mfma_f32_64x64s2"),
                                           ("f32", "mfma_f32_64x64s4"), ("f32", "mfma_f32_32x32s4"), ("f32", "mfma_f32_128x128s2"), ("f64", "mfma_f64_64x64s2"), ("f64", "mfma_f64_32x32s4"), ("f32", "mfma_f32_128x128"),
                                           ("f32", "mfma_f32_256x128"), ("f64", "auto"), ("f64", "mfma_f64_64x64"),
                                           ("f64", "mfma_f64_128x64"), ("f64", "mfma_f64_128x128"), ("f32", "tile64"),
                                           ("f32", "mfma_f32_256x128d"), ("f32", "mfma_f32_128x128d"), ("f32", "mfma_f32_64x64d"),
                                           ("f64", "mfma_f64_128x128d"), ("f64", "mfma_f64_64x64d")])
@pytest.mark.parametrize("kind", ["none", "sigmoid", "tanh"])
def test_fused_equals_two_calls(dev, dtype, variant, kind):
    assert dev.lib.wk_gemm_force_variant(variant.encode()) == 0
    try:
        seed = 0
        for (M, N, K, extra) in [(256, 256, 64, 0), (128, 384, 100, 0), (70, 45, 33, 0), (257, 129, 17, 3), (300, 200, 96, 4),
                                 (512, 256, 48, 4), (256, 128, 16, 0), (768, 384, 160, 8)]:
            for with_bias in (True, False):
                seed += 1
                fused, two, A, B, bias = both(dev, dtype, M, N, K, 0, 1, kind, with_bias, seed, extra)
                assert np.array_equal(fused, two), f"{M}x{N}x{K} bias={with_bias}"
                # and against the float64 restatement
                z = A.astype(np.float64) @ B.astype(np.float64) + (bias.astype(np.float64) if bias is not None else 0.0)
                want = {"none": z, "sigmoid": 1 / (1 + np.exp(-z)), "tanh": np.tanh(z)}[kind]
                eps = np.finfo(oracle.real_np_dtype(dtype)).eps
                assert np.abs(fused - want).max() <= 8 * eps * np.sqrt(K) * max(1.0, np.abs(z).max())
    finally:
        dev.lib.wk_gemm_force_variant(b"auto")


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("op_a,op_b", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("kind", ["none", "sigmoid", "tanh"])
def test_fused_small_batches(dev, dtype, op_a, op_b, kind):
    """A batch of at most 32 rows through a large weight matrix, and a large batch into at most 32 outputs: the
    kernel for such products carries the bias and the activation in every layout (the bias goes by the column
    of C whichever side is the short one).  Against the two calls to the bit and against float64."""
    did = raw.dtype_id(dtype)
    per = 16 // np.dtype(oracle.real_np_dtype(dtype)).itemsize
    seed = 40
    for (M, N, K) in [(32, 4096, 2048), (7, 4100, 1100), (4096, 24, 2052), (20, 1024, 4100)]:
        assert dev.lib.wk_gemm_variant(did, op_a, op_b, M, N, K, M if op_a else K, K if op_b else N, N, None, None, None) == b"skinny"
        for with_bias in (True, False):
            seed += 1
            fused, two, A, B, bias = both(dev, dtype, M, N, K, op_a, op_b, kind, with_bias, seed, per if with_bias else 0)
            assert np.array_equal(fused, two), f"{M}x{N}x{K} bias={with_bias}"
            z = A.astype(np.float64) @ B.astype(np.float64) + (bias.astype(np.float64) if bias is not None else 0.0)
            want = {"none": z, "sigmoid": 1 / (1 + np.exp(-z)), "tanh": np.tanh(z)}[kind]
            eps = np.finfo(oracle.real_np_dtype(dtype)).eps
            assert np.abs(fused - want).max() <= 8 * eps * np.sqrt(K) * max(1.0, np.abs(z).max())


@pytest.mark.parametrize("op_a,op_b", [(0, 0), (1, 0), (1, 1)])
def test_other_layouts_run_the_two_calls(dev, op_a, op_b):
    fused, two, _A, _B, _bias = both(dev, "f32", 130, 70, 50, op_a, op_b, "tanh", True, 9)
    assert np.array_equal(fused, two)


def test_fused_invalid_arguments(dev):
    buf = dev.malloc(4096)
    p, lib = buf.ptr, dev.lib
    f32 = raw.dtype_id("f32")
    assert lib.wk_gemm_bias_activation(dev.stream, f32, 0, 1, 4, 4, 4, p, 4, p, 4, p, 4, None, 2) == 1          # unknown activation
    assert lib.wk_gemm_bias_activation(dev.stream, raw.dtype_id("i32"), 0, 1, 4, 4, 4, p, 4, p, 4, p, 4, None, -1) == 9
    assert lib.wk_gemm_bias_activation(dev.stream, f32, 0, 1, 4, 4, 4, p, 3, p, 4, p, 4, None, -1) == 1          # lda < K
    assert lib.wk_gemm_bias_activation(dev.stream, f32, 0, 1, 0, 4, 4, p, 4, p, 4, p, 4, None, -1) == 1
    buf.free()
