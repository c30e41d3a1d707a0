"""GPU: tensor.printZ through the mirrored API against texts written out by hand from the layout
rules of src/tensor/print.zig (printVector :103-217, printVectorOrMatrix :219-264, printDim :266-314,
printZ :316-361).  The reference holds no expected text for print (its test block only calls it), so
these strings follow its code, not a recorded output: parity of the number formatting with Zig's
`{d}` / `{e}` is unpinned."""
import numpy as np
import pytest

import oracle
from wekua_amd import Context, DeviceType, Pipeline, Tensor, memory, printZ

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    context = Context.initFromDeviceType(DeviceType.all)
    pipeline = Pipeline.init(context.command_queues[0])
    yield context, pipeline
    pipeline.deinit()
    context.deinit()


def text_of(env, dtype, values):
    context, pipeline = env
    host = np.asarray(values, dtype=oracle.real_np_dtype(dtype))
    shape = host.shape[:-1] if oracle.is_complex(dtype) else host.shape
    t = Tensor.alloc(dtype, context, pipeline, shape)
    memory.readFromBuffer(pipeline, t, host)
    out = printZ(pipeline, t)
    t.release(pipeline)
    return out


def f(v):   # "{d: >14.8}," / "{e: >14.5},"
    return v.rjust(14) + ","


def test_f32_vector_fixed_and_scientific(env):
    got = text_of(env, "f32", [1, -2.5, 10000, 0.3])
    want = "Tensor([" + f("1.00000000") + f("-2.50000000") + f("1.00000e4") + f("0.30000000") + "], shape=(4), dtype=f32)\n"
    assert got == want


def test_f64_vector_elision(env):
    # 9 columns: all shown (4 head, dec = 5); 10 columns: 4, "...", last 4
    got9 = text_of(env, "f64", np.arange(9))
    assert got9 == "Tensor([" + "".join(f(f"{i}.00000000") for i in range(9)) + "], shape=(9), dtype=f64)\n"
    got10 = text_of(env, "f64", np.arange(10))
    items = [f(f"{i}.00000000") for i in range(4)] + [f("...")] + [f(f"{i}.00000000") for i in range(6, 10)]
    assert got10 == "Tensor([" + "".join(items) + "], shape=(10), dtype=f64)\n"


def test_i32_matrix(env):
    def i(v):
        return str(v).rjust(12) + ","   # len("-2147483648") + 1
    got = text_of(env, "i32", [[1, 2], [3, -4]])
    want = "Tensor([\n  " + i(1) + i(2) + "\n  " + i(3) + i(-4) + "\n], shape=(2, 2), dtype=i32)\n"
    assert got == want
    # 6 columns > max_items = 5: two, "...", two
    got = text_of(env, "i32", np.arange(6))
    assert got == "Tensor([" + i(0) + i(1) + i("...") + i(4) + i(5) + "], shape=(6), dtype=i32)\n"
    got = text_of(env, "i32", np.arange(5))
    assert got == "Tensor([" + "".join(i(v) for v in range(5)) + "], shape=(5), dtype=i32)\n"


def test_u8_rows_elision(env):
    def i(v):
        return str(v).rjust(4) + ","    # len("255") + 1; max_items = 21, ten leading items
    rows = np.arange(6 * 3).reshape(6, 3)
    got = text_of(env, "u8", rows)
    line = lambda r: "\n  " + "".join(i(v) for v in rows[r])
    want = "Tensor([" + line(0) + line(1) + "\n   ... " + line(4) + line(5) + "\n], shape=(6, 3), dtype=u8)\n"
    assert got == want
    got = text_of(env, "u8", np.arange(23))
    items = [i(v) for v in range(10)] + [i("...")] + [i(v) for v in range(13, 23)]
    assert got == "Tensor([" + "".join(items) + "], shape=(23), dtype=u8)\n"


def test_three_dimensions(env):
    vals = np.arange(5 * 1 * 2).reshape(5, 1, 2)
    got = text_of(env, "f64", vals)

    def block(k):
        return "  [\n    " + f(f"{vals[k, 0, 0]}.00000000") + f(f"{vals[k, 0, 1]}.00000000") + "\n  ],\n"
    want = "Tensor([\n" + block(0) + block(1) + "\n  ... \n" + block(3) + block(4) + "\n], shape=(5, 1, 2), dtype=f64)\n"
    assert got == want


def test_complex(env):
    def c(v):
        return v.rjust(24) + ","
    got = text_of(env, "cf32", [[1, 2], [0, 3], [4, 0], [0, 0], [-1.5, -0.25], [2, 2]])
    items = [c("1.00e0+2.00e0j"), c("3.00000e0j"), c("..."), c("-1.50e0-2.50e-1j"), c("2.00e0+2.00e0j")]
    assert got == "Tensor([" + "".join(items) + "], shape=(6), dtype=complex_f32)\n"
    got = text_of(env, "cf64", [[4, 0], [0, 0]])
    assert got == "Tensor([" + c("4.00000e0") + c("0.00000e0") + "], shape=(2), dtype=complex_f64)\n"

    def ci(v):
        return v.rjust(10) + ","    # len("-128-128j") + 1; max_items = 7, three leading items
    got = text_of(env, "ci8", [[1, 2], [3, -4], [0, 5], [6, 0], [0, 0]])
    assert got == "Tensor([" + ci("1+2j") + ci("3-4j") + ci("5j") + ci("6") + ci("0") + "], shape=(5), dtype=complex_i8)\n"
