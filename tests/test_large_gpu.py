"""GPU: element counts and byte offsets beyond 2^32 -- the sizes a 288 GB device invites and the ones
where a 32-bit index anywhere in a kernel shows.  Inputs are made on the device by random.uniform,
whose value at any logical index the oracle gives (oracle/tensor_ops.py hash64), so windows of the
big tensors can be checked without the host ever holding them: the start, both sides of element
2^30 (byte offset 4 GiB for f32) and 2^31, and the tail.  About 20 GB of device memory."""
import ctypes

import numpy as np
import pytest

import oracle
import wekua_amd as wk
from oracle import tensor_ops as ot
from wekua_amd import _capi, raw

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    context = wk.Context.initFromDeviceType(wk.DeviceType.all)
    pipeline = wk.Pipeline.init(context.command_queues[0])
    rawdev = raw.Device(0)                  # a second stream, for copying windows out of the big buffers
    yield context, pipeline, rawdev
    rawdev.close()
    pipeline.deinit()
    context.deinit()


def window(env, tensor, start, count, np_dtype):
    """Elements [start, start + count) of a dense 1-D tensor, copied straight from its buffer."""
    _context, pipeline, rawdev = env
    out = np.empty(count, dtype=np_dtype)
    src = ctypes.c_void_p(tensor.buffer + start * out.itemsize)
    pipeline.waitAndCleanup()
    _capi.check(rawdev.lib.wk_copy_d2h_rect_async(rawdev.stream, out.ctypes.data, out.nbytes, out.nbytes, src, out.nbytes,
                                                  out.nbytes, out.nbytes, 1, 1), "copy")
    rawdev.sync()
    return out


def expected_uniform(seed, start, count):
    idx = np.arange(start, start + count, dtype=np.uint64)
    return ot._component(ot.hash64(idx, seed), np.dtype(np.float32), None, None)


def test_axpy_and_uniform_beyond_2_pow_31_elements(env):
    context, pipeline, _rawdev = env
    n = 2 ** 31 + 4099                      # 8.6 GB per f32 vector; odd tail for the element-wise remainder
    x = wk.Tensor.alloc("f32", context, pipeline, (n,))
    y = wk.Tensor.alloc("f32", context, pipeline, (n,))
    wk.random.uniform(pipeline, x, 11)
    wk.random.uniform(pipeline, y, 12)
    windows = [(0, 4096), (2 ** 30 - 2048, 4096), (2 ** 31 - 2048, 4096), (n - 4099, 4099)]
    for start, count in windows:            # the generator itself at 64-bit indices
        assert np.array_equal(window(env, x, start, count, np.float32), expected_uniform(11, start, count))
        assert np.array_equal(window(env, y, start, count, np.float32), expected_uniform(12, start, count))
    wk.blas.axpy(pipeline, x, 0.75, y)
    for start, count in windows:
        xe, ye = expected_uniform(11, start, count), expected_uniform(12, start, count)
        want = oracle.axpy("f32", xe, 0.75, ye, contract=True)
        assert np.array_equal(window(env, y, start, count, np.float32), want), f"window at {start}"
    x.release(pipeline)
    y.release(pipeline)


def test_gemm_operand_beyond_4_gib(env):
    """A is 65536 x 16400 f32 (4.3 GB, so the last rows start beyond byte offset 2^32), B is
    16400 x 256: every row block of C is checked on sampled rows against float64 dot products of the
    same generated values."""
    context, pipeline, _rawdev = env
    M, K, N = 65536, 16400, 256
    a = wk.Tensor.alloc("f32", context, pipeline, (M, K))
    b = wk.Tensor.alloc("f32", context, pipeline, (K, N))
    c = wk.Tensor.alloc("f32", context, pipeline, (M, N))
    assert a.row_pitch == K                 # dense: the logical index is the buffer index
    wk.random.uniform(pipeline, a, 21)
    wk.random.uniform(pipeline, b, 22)
    wk.blas.gemm(pipeline, None, a, 0, b, 0, None, c, None)
    got = np.empty((M, N), dtype=np.float32)
    wk.memory.writeToBuffer(pipeline, c, got)
    pipeline.waitAndCleanup()
    bh = expected_uniform(22, 0, K * N).reshape(K, N).astype(np.float64)
    rows = np.array([0, 1, 255, 256, 32767, 32768, 65279, 65280, 65472, 65473, 65534, 65535])
    assert 65472 * K * 4 < 2 ** 32 < 65473 * K * 4     # the byte offset of a row start crosses 4 GiB here
    for r in rows:
        ar = expected_uniform(21, int(r) * K, K).astype(np.float64)
        want = ar @ bh
        bound = np.abs(ar) @ np.abs(bh)
        err = np.abs(got[r].astype(np.float64) - want) / bound
        assert err.max() <= 1e-5 * np.sqrt(K), f"row {r}: {err.max():.3e}"
    for t in (a, b, c):
        t.release(pipeline)


def test_int32_gemm_packed_planes_beyond_4_gib(env):
    """int32 65536 x 16400 times 16400 x 1024 through blas.gemm with a GemmPackedTensors: the product is
    large enough for the pack pass, whose digit planes of A alone are 4.3 GB.  Entries are the low 32
    bits of the generator's hash (full range, so every sum wraps); sampled rows are compared bit for
    bit with int64 arithmetic reduced modulo 2^32."""
    context, pipeline, _rawdev = env
    M, K, N = 65536, 16400, 1024
    a = wk.Tensor.alloc("i32", context, pipeline, (M, K))
    b = wk.Tensor.alloc("i32", context, pipeline, (K, N))
    c = wk.Tensor.alloc("i32", context, pipeline, (M, N))
    assert a.row_pitch == K and b.row_pitch == N
    wk.random.uniform(pipeline, a, 31)
    wk.random.uniform(pipeline, b, 32)
    packed = wk.GemmPackedTensors.init(pipeline, c, K, True)
    assert packed.workspace_bytes > 2 ** 32
    name = _capi.load().wk_gemm_variant_with_workspace(raw.dtype_id("i32"), 0, 0, M, N, K, K, N, N, a.buffer, b.buffer,
                                                       c.buffer, packed.workspace_bytes)
    assert name == b"mfma_i32_packed"
    wk.blas.gemm(pipeline, 3, a, 0, b, 0, None, c, packed)
    got = np.empty((M, N), dtype=np.int32)
    wk.memory.writeToBuffer(pipeline, c, got)
    pipeline.waitAndCleanup()

    def ints(seed, start, count):
        idx = np.arange(start, start + count, dtype=np.uint64)
        return ot._component(ot.hash64(idx, seed), np.dtype(np.int32), None, None).astype(np.int64)
    bh = ints(32, 0, K * N).reshape(K, N)
    for r in (0, 127, 128, 32768, 65472, 65473, 65535):
        with np.errstate(over="ignore"):
            want = ((ints(31, r * K, K) @ bh) * 3) & 0xFFFFFFFF
        assert np.array_equal(got[r].view(np.uint32).astype(np.int64), want), f"row {r}"
    packed.deinit(pipeline)
    for t in (a, b, c):
        t.release(pipeline)


def test_transpose_and_copy_beyond_4_gib(env):
    """transpose of a 32768 x 40000 f32 tensor (5.2 GB) into a skew-pitched 40000 x 32768 one, and
    memory.copy of the result: sampled rows of both against the generator's values."""
    context, pipeline, _rawdev = env
    R, C = 32768, 40000
    src = wk.Tensor.alloc("f32", context, pipeline, (R, C))
    dst = wk.Tensor.alloc("f32", context, pipeline, (C, R))
    wk.random.uniform(pipeline, src, 41)
    wk.transpose(pipeline, dst, src, 0, 1)
    rows = (0, 1, 20000, 32000, 39998, 39999)          # row j of dst starts at byte j * pitch * 4: beyond 2^32 from j = 32641
    assert 32000 * dst.row_pitch * 4 < 2 ** 32 < 39998 * dst.row_pitch * 4

    def check(tensor):
        for j in rows:
            got = window(env, tensor, j * tensor.row_pitch, R, np.float32)
            idx = np.arange(R, dtype=np.uint64) * np.uint64(C) + np.uint64(j)     # src[i][j]
            want = ot._component(ot.hash64(idx, 41), np.dtype(np.float32), None, None)
            assert np.array_equal(got, want), f"row {j}"
    check(dst)
    src.release(pipeline)
    dup = wk.Tensor.alloc("f32", context, pipeline, (C, R))
    wk.memory.copy(pipeline, dst, dup)
    check(dup)
    dst.release(pipeline)
    dup.release(pipeline)
