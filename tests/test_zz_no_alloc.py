"""GPU: wk_bias_step_static -- the entry point for callers that cannot allocate -- against
wk_bias_step, through the C ABI.  Both run the same kernels with equally sized partial buffers, so
the results must agree bit for bit.  Each case makes two calls in a row on the one per-device array,
the second with a smaller input, so that partials left over from the first call would show."""

import numpy as np
import pytest

from wekua_amd import raw, synth

pytestmark = pytest.mark.gpu

DT = {"f32": np.float32, "f64": np.float64}


def both(dev, dtype, rows, cols, pitch, seed):
    host = np.full((rows, pitch), 1e30, dtype=DT[dtype])        # gaps poisoned: they must not be summed
    host[:, :cols] = synth.uniform(seed, (rows, cols), DT[dtype])
    sens = dev.upload(host)
    out_a = dev.upload(np.full(cols + 8, -7.0, dtype=DT[dtype]))
    out_b = dev.upload(np.full(cols + 8, -7.0, dtype=DT[dtype]))
    did = raw.dtype_id(dtype)
    rc = dev.lib.wk_bias_step(dev.stream, did, rows, cols, sens.ptr, pitch, out_a.ptr)
    assert rc == 0, rc
    rc = dev.lib.wk_bias_step_static(dev.stream, did, rows, cols, sens.ptr, pitch, out_b.ptr)
    assert rc == 0, rc
    dev.sync()
    a = out_a.download(DT[dtype], (cols + 8,))
    b = out_b.download(DT[dtype], (cols + 8,))
    for buf in (sens, out_a, out_b):
        buf.free()
    assert (b[cols:] == -7.0).all(), "wrote past the last column"
    # and against the column sums themselves (float64 on the host), so that "equal" is not "equally wrong"
    want = host[:, :cols].astype(np.float64).sum(axis=0)
    bound = np.abs(host[:, :cols]).astype(np.float64).sum(axis=0) * rows * np.finfo(DT[dtype]).eps
    assert np.all(np.abs(b[:cols] - want) <= bound + 1e-300)
    return a[:cols], b[:cols]


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("first,second", [
    ((2048, 4096, 4096), (300, 1000, 1004)),     # configuration 5's widest layer, then fewer bands and columns
    ((4099, 777, 780), (40, 130, 136)),          # ragged, then two bands only
    ((5000, 20000, 20000), (33, 5, 8)),          # bands limited by the array's size, then a tiny case
    ((64, 64, 64), (7, 3, 4)),                   # second call takes one band and never touches the array
])
def test_static_scratch_equals_stream_scratch_on_two_calls_in_a_row(dev, dtype, first, second):
    for i, (rows, cols, pitch) in enumerate((first, second)):
        a, b = both(dev, dtype, rows, cols, pitch, 0xB1A5 + i)
        assert np.array_equal(a, b), f"{dtype} call {i}: rows={rows} cols={cols}"


def test_static_scratch_limits_and_errors(dev):
    lib = dev.lib
    buf = dev.malloc(1 << 16)
    f32, f64 = raw.dtype_id("f32"), raw.dtype_id("f64")
    limit = 1 << 20
    # a row of partials may take at most half the array; the pointer is not touched before the check
    assert lib.wk_bias_step_static(dev.stream, f32, 4, limit // 2 // 4 + 1, buf.ptr, limit, buf.ptr) == 11
    assert lib.wk_bias_step_static(dev.stream, f64, 4, limit // 2 // 8 + 1, buf.ptr, limit, buf.ptr) == 11
    assert b"ScratchTooSmall" in lib.wk_strerror(11)
    assert lib.wk_bias_step_static(dev.stream, raw.dtype_id("i32"), 4, 4, buf.ptr, 4, buf.ptr) == 9
    assert lib.wk_bias_step_static(dev.stream, f32, 0, 4, buf.ptr, 4, buf.ptr) == 1
    assert lib.wk_bias_step_static(dev.stream, f32, 4, 8, buf.ptr, 4, buf.ptr) == 1      # pitch < cols
    assert lib.wk_bias_step_static(dev.stream, f32, 4, 4, None, 4, buf.ptr) == 1
    buf.free()


def test_static_scratch_at_its_column_limit(dev):
    """The widest row the array takes (131072 f32 columns: two bands of partials fill it exactly)."""
    cols = (1 << 20) // 2 // 4
    a, b = both(dev, "f32", 70, cols, cols, 0xB1B0)
    assert np.array_equal(a, b)
    a, b = both(dev, "f32", 9, 17, 20, 0xB1B1)
    assert np.array_equal(a, b)
