"""GPU: the MLP training step (math.dot / sum / mean, activations, Linear, Sequential, Cache,
loss.mse, GD and Adam) through the reference-shaped API, against the numpy restatement
(oracle/nn.py) and the reference's own known answers.

Tolerances (relative to the magnitude named in each assertion):
  * element-wise kernels whose arithmetic is fixed (mse, sigmoid_dev, hadamard): exact;
    tanh_dev 1 - y*y may be contracted into one fused multiply-add: 1 eps
  * exp / tanh: 8 eps (the device's math library versus numpy's)
  * sums over n terms: n * eps * sum|x| (the order of summation is free)
  * whole-network quantities in f32 against the float64 restatement: 1e-5 * sqrt(K) of the
    operand magnitude, the bound the gemm tests use, accumulated over the layers
"""
import numpy as np
import pytest

import wekua_amd as wk
from oracle import nn as onn
from wekua_amd import Context, DeviceType, Pipeline, Tensor, memory, nn, synth

pytestmark = pytest.mark.gpu

NP = {"f32": np.float32, "f64": np.float64}
ACT = {onn.SIGMOID: nn.Sigmoid, onn.TANH: nn.Tanh}


@pytest.fixture(scope="module")
def env():
    context = Context.initFromDeviceType(DeviceType.all)
    pipeline = Pipeline.init(context.command_queues[0])
    yield context, pipeline
    pipeline.deinit()
    context.deinit()


def upload(context, pipeline, dtype, host):
    t = Tensor.alloc(dtype, context, pipeline, host.shape)
    memory.readFromBuffer(pipeline, t, host)
    return t


def download(pipeline, t):
    out = np.empty(t.shape, dtype=NP[t.dtype])
    memory.writeToBuffer(pipeline, t, out)
    pipeline.waitAndCleanup()
    return out


# ---- the reference's own known answers -----------------------------------------------------------

@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_math_known_answers(env, dtype):
    context, pipeline = env
    dt = NP[dtype]
    # src/math/basic.zig:258-320
    x = upload(context, pipeline, dtype, np.arange(1, 5, dtype=dt))
    y = upload(context, pipeline, dtype, np.arange(2, 6, dtype=dt))
    wk.math.dot(pipeline, x, y)
    assert np.array_equal(download(pipeline, x), np.array([2, 6, 12, 20], dtype=dt))
    # src/math/basic.zig:322-366
    s = upload(context, pipeline, dtype, np.arange(1, 6, dtype=dt))
    assert wk.math.sum(pipeline, s) == dt(15)
    # src/math/basic.zig:368-420
    m = upload(context, pipeline, dtype, np.array([2, 4, 6, 8], dtype=dt))
    assert abs(float(wk.math.mean(pipeline, m)) - 5.0) < 1e-5
    # src/math/trig.zig:397-450 (through the Tanh activation, which is what calls it)
    t = upload(context, pipeline, dtype, np.array([0, 1], dtype=dt))
    nn.Tanh.init().run(pipeline, t)
    got = download(pipeline, t)
    assert abs(float(got[0])) < 1e-4 and abs(float(got[1]) - 0.7616) < 1e-4
    for z in (x, y, s, m, t):
        z.release(pipeline)


def test_shape_mismatch_is_rejected(env):
    context, pipeline = env
    x = Tensor.alloc("f32", context, pipeline, (4, 3))
    y = Tensor.alloc("f32", context, pipeline, (3, 4))
    with pytest.raises(wk.WekuaError) as e:
        wk.math.dot(pipeline, x, y)
    assert e.value.name == "UnqualTensorsShape"
    i8 = Tensor.alloc("i8", context, pipeline, (4,))
    with pytest.raises(wk.WekuaError) as e:
        wk.math.dot(pipeline, i8, i8)
    assert e.value.name == "TypeNotSupported"
    for t in (x, y, i8):
        t.release(pipeline)


# ---- kernels against the restatement -----------------------------------------------------------------

SHAPES = [(1,), (7,), (5, 3), (33, 65), (3, 17, 19), (64, 1024), (129, 2048)]


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("shape", SHAPES)
def test_elementwise_kernels(env, dtype, shape):
    context, pipeline = env
    dt = NP[dtype]
    eps = np.finfo(dt).eps
    xh = synth.uniform(11, shape, dt, -4.0, 4.0)
    yh = synth.uniform(12, shape, dt)
    # math.dot
    x, y = upload(context, pipeline, dtype, xh), upload(context, pipeline, dtype, yh)
    wk.math.dot(pipeline, x, y)
    assert np.array_equal(download(pipeline, x), onn.hadamard(xh, yh))
    assert np.array_equal(download(pipeline, y), yh)  # the second operand is read only
    for kind in (onn.SIGMOID, onn.TANH):
        act = ACT[kind].init()
        a = upload(context, pipeline, dtype, xh)
        d = Tensor.alloc(dtype, context, pipeline, shape)
        act.run(pipeline, a)
        got = download(pipeline, a)
        want = onn.activation(kind, xh)
        assert np.allclose(got, want, rtol=8 * eps, atol=eps), f"activation {kind} {shape}"
        act.getDerivative(pipeline, a, d)
        gd = download(pipeline, d)
        wd = onn.activation_dev(kind, got)  # from the device's own activation output
        assert np.allclose(gd, wd, rtol=0, atol=eps if kind == onn.TANH else 0), f"derivative {kind} {shape}"
        assert np.array_equal(download(pipeline, a), got)  # the output is read only
        a.release(pipeline)
        d.release(pipeline)
    # sum / mean
    n = xh.size
    tol = n * eps * float(np.abs(xh.astype(np.float64)).sum())
    x2 = upload(context, pipeline, dtype, xh)
    exact = float(xh.astype(np.float64).sum())
    assert abs(float(wk.math.sum(pipeline, x2)) - exact) <= tol + 1e-300
    assert abs(float(wk.math.mean(pipeline, x2)) - exact / n) <= tol / n + eps * abs(exact / n)
    assert abs(float(onn.tensor_sum(xh)) - exact) <= tol + 1e-300  # the restatement, same bound
    for t in (x, y, x2):
        t.release(pipeline)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("rows,cols", [(1, 1), (4, 1), (19, 11), (64, 256), (2048, 1000), (1000, 4096)])
def test_mse_bias_and_bias_step(env, dtype, rows, cols):
    context, pipeline = env
    dt = NP[dtype]
    eps = np.finfo(dt).eps
    oh = synth.uniform(21, (rows, cols), dt)
    eh = synth.uniform(22, (rows, cols), dt, 0.0, 1.0)
    bh = synth.uniform(23, (cols,), dt)
    # a one-matrix layer exposes its cache tensors; loss.mse writes error and last sensitivity
    layer = nn.Linear.init(dtype, context, pipeline, 3, cols, nn.Sigmoid.init(), seed=1)
    cache = nn.Cache.init(context, pipeline, rows, [layer])
    lc = cache.getLayerCache(0)
    out, exp = upload(context, pipeline, dtype, oh), upload(context, pipeline, dtype, eh)
    nn.loss.mse(True, pipeline, out, exp, cache, None)
    want_err, want_dev = onn.mse(oh, eh)
    assert np.array_equal(download(pipeline, cache.error_tensor), want_err)
    assert np.array_equal(download(pipeline, layer.getSensitivity(lc)), want_dev)
    res = np.zeros(1, dtype=dt)
    nn.loss.mse(False, pipeline, out, exp, cache, res)
    exact = float(want_err.astype(np.float64).mean())
    assert abs(float(res[0]) - exact) <= rows * cols * eps * exact + 1e-300
    # bias + activation through forward: weights zeroed, so forward = act(bias)
    w = layer.getWeights()[0]
    wk.fill.zeroes(pipeline, w)
    memory.readFromBuffer(pipeline, layer.getBias()[0], bh)
    x = upload(context, pipeline, dtype, synth.uniform(24, (rows, 3), dt))
    got = download(pipeline, layer.forward(pipeline, x, lc))
    want = onn.activation(onn.SIGMOID, onn.bias_add(np.zeros((rows, cols), dt), bh))
    assert np.allclose(got, want, rtol=8 * eps, atol=eps)
    # bias_step: backward's bias gradient is the column sum of (sensitivity * derivative)
    memory.readFromBuffer(pipeline, layer.getSensitivity(lc), oh)
    layer.backward(pipeline, lc, x, None)
    sens = onn.hadamard(oh, onn.activation_dev(onn.SIGMOID, got))
    want_bg = onn.bias_step(sens)
    got_bg = download(pipeline, layer.getBiasGradients(lc)[0])
    bound = rows * eps * np.abs(sens.astype(np.float64)).sum(axis=0) + 1e-300
    assert np.all(np.abs(got_bg.astype(np.float64) - sens.astype(np.float64).sum(axis=0)) <= bound)
    assert np.all(np.abs(want_bg.astype(np.float64) - sens.astype(np.float64).sum(axis=0)) <= bound)
    for t in (out, exp, x):
        t.release(pipeline)
    cache.deinit(pipeline)
    layer.deinit(pipeline)


# ---- the network -----------------------------------------------------------------------------------------

def build_network(context, pipeline, dtype, sizes, acts, deep=1, bias=True, seed=7):
    seq = nn.Sequential.init(dtype)
    for i, ((n_in, n_out), act) in enumerate(zip(zip(sizes[:-1], sizes[1:]), acts)):
        seq.append(nn.Linear.init(dtype, context, pipeline, n_in, n_out, ACT[act].init() if act is not None else None,
                                  deep=deep, enable_bias=bias, seed=seed + i))
    return seq


def host_layers(pipeline, seq, acts, deep, as_dtype):
    """Device weights and biases as the oracle's layer list (cast to `as_dtype`)."""
    ws = [download(pipeline, w).astype(as_dtype) for w in seq.getWeights()]
    bs = [download(pipeline, b).astype(as_dtype) if b is not None else None for b in seq.getBias()]
    return [{"w": ws[i * deep:(i + 1) * deep], "b": bs[i * deep:(i + 1) * deep], "act": a} for i, a in enumerate(acts)]


def close(got, want, k, dtype, what):
    """|got - want| <= tol * sqrt(k) * max|want| with the gemm tests' per-dtype tol."""
    tol = {"f32": 1e-5, "f64": 1e-12}[dtype] * np.sqrt(k)
    scale = float(np.abs(want).max()) + 1e-30
    err = float(np.abs(got.astype(np.float64) - want).max())
    assert err <= tol * scale, f"{what}: err {err:.3e} > {tol * scale:.3e}"


def test_xavier_initialisation(env):
    context, pipeline = env
    layer = nn.Linear.init("f32", context, pipeline, 300, 200, None, deep=2, seed=5)
    w0, w1 = (download(pipeline, w) for w in layer.getWeights())
    assert w0.shape == (200, 300) and w1.shape == (200, 200)
    for w, (i, o) in ((w0, (300, 200)), (w1, (200, 200))):
        limit = np.sqrt(6.0 / (i + o))  # getRandomLimits, src/nn/layer/linear.zig:28-45
        assert np.abs(w).max() <= limit and np.abs(w).max() > 0.98 * limit
        assert abs(float(w.mean())) < 0.02 * limit and abs(float(w.std()) - limit / np.sqrt(3)) < 0.02 * limit
    assert all(not download(pipeline, b).any() for b in layer.getBias())
    again = nn.Linear.init("f32", context, pipeline, 300, 200, None, deep=2, seed=5)
    assert np.array_equal(download(pipeline, again.getWeights()[0]), w0)  # seeded: repeatable
    unseeded = nn.Linear.init("f32", context, pipeline, 300, 200, None)
    assert not np.array_equal(download(pipeline, unseeded.getWeights()[0]), w0)
    for l in (layer, again, unseeded):
        l.deinit(pipeline)
    with pytest.raises(wk.WekuaError) as e:
        nn.Linear.init("f32", context, pipeline, 0, 4, None)
    assert e.value.name == "InvalidValue"


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("deep,bias", [(1, True), (2, True), (1, False)])
def test_training_step_gd(env, dtype, deep, bias):
    context, pipeline = env
    dt = NP[dtype]
    sizes, acts, batch = [37, 53, 29, 11], [onn.TANH, onn.TANH, onn.SIGMOID], 19
    seq = build_network(context, pipeline, dtype, sizes, acts, deep=deep, bias=bias)
    layers = host_layers(pipeline, seq, acts, deep, np.float64)
    xh = synth.normal(31, (batch, sizes[0]), dt)
    yh = synth.uniform(32, (batch, sizes[-1]), dt, 0.0, 1.0)
    x, y = upload(context, pipeline, dtype, xh), upload(context, pipeline, dtype, yh)
    cache = nn.Cache.init(context, pipeline, batch, [seq])
    lc = cache.getLayerCache(0)
    opt = nn.optimizers.GD.init(dtype, 0.05)

    out = seq.forward(pipeline, x, lc)
    loss = np.zeros(1, dtype=dt)
    nn.loss.mse(True, pipeline, out, y, cache, loss)
    seq.backward(pipeline, lc, x, None)
    got_out = download(pipeline, out)
    got_g = [download(pipeline, g) for g in seq.getGradients(lc)]
    got_bg = [download(pipeline, g) if g is not None else None for g in seq.getBiasGradients(lc)]
    opt.step(pipeline, cache)
    got_w = [download(pipeline, w) for w in seq.getWeights()]

    want_out, want_err, want_grads, _ = onn.mlp_step(xh.astype(np.float64), yh.astype(np.float64), layers, ("gd", 0.05))
    k = max(sizes) * len(sizes)
    close(got_out, want_out, k, dtype, "output")
    assert abs(float(loss[0]) - want_err.mean()) <= {"f32": 1e-5, "f64": 1e-12}[dtype] * np.sqrt(k)
    flat_g = [g for lg, _ in want_grads for g in lg]
    flat_bg = [g for _, lbg in want_grads for g in lbg]
    for i, (g, wg) in enumerate(zip(got_g, flat_g)):
        close(g, wg, k * batch, dtype, f"gradient {i}")
    for i, (g, wg) in enumerate(zip(got_bg, flat_bg)):
        assert (g is None) == (wg is None)
        if g is not None:
            close(g, wg, k * batch, dtype, f"bias gradient {i}")
    flat_w = [w for l in layers for w in l["w"]]
    for i, (w, ww) in enumerate(zip(got_w, flat_w)):
        close(w, ww, k * batch, dtype, f"updated weight {i}")
    opt.deinit(pipeline)
    cache.deinit(pipeline)
    seq.deinit(pipeline)
    x.release(pipeline)
    y.release(pipeline)


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_adam_kernel_and_closed_form(env, dtype):
    """One parameter tensor under a constant known gradient: drive the optimizer through a layer
    whose gradient tensors are written by hand."""
    context, pipeline = env
    dt = NP[dtype]
    eps_m = np.finfo(dt).eps
    layer = nn.Linear.init(dtype, context, pipeline, 40, 30, nn.Tanh.init(), seed=3)
    cache = nn.Cache.init(context, pipeline, 5, [layer])
    lc = cache.getLayerCache(0)
    w0 = download(pipeline, layer.getWeights()[0])
    b0 = download(pipeline, layer.getBias()[0])
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    opt = nn.optimizers.Adam.init(dtype, lr, b1, b2, eps)
    w, b = w0.copy(), b0.copy()
    mw = vw = np.zeros_like(w0)
    mb = vb = np.zeros_like(b0)
    for t in range(1, 6):
        gw = synth.uniform(40 + t, w0.shape, dt, -2.0, 2.0)
        gb = synth.uniform(50 + t, b0.shape, dt, -2.0, 2.0)
        memory.readFromBuffer(pipeline, layer.getGradients(lc)[0], gw)
        memory.readFromBuffer(pipeline, layer.getBiasGradients(lc)[0], gb)
        opt.step(pipeline, cache)
        w_prev = w
        w, mw, vw = onn.adam_update(w, gw, mw, vw, lr, b1, b2, eps, t)
        b, mb, vb = onn.adam_update(b, gb, mb, vb, lr, b1, b2, eps, t)
        got_w = download(pipeline, layer.getWeights()[0])
        got_b = download(pipeline, layer.getBias()[0])
        # the update is at most ~lr per step; compare the updates to a few ulp of the parameters
        assert np.allclose(got_w, w, rtol=0, atol=4 * eps_m * (np.abs(w0).max() + t * lr)), f"step {t}"
        assert np.allclose(got_b, b, rtol=0, atol=4 * eps_m * (np.abs(b0).max() + t * lr) + 1e-30), f"step {t}"
        if t == 1:  # closed form of the first step: dw = -lr * g / (|g| + eps)
            g64 = gw.astype(np.float64)
            want = w_prev.astype(np.float64) - lr * g64 / (np.abs(g64) + eps)
            assert np.allclose(got_w, want, rtol=0, atol=4 * eps_m * np.abs(w0).max())
    opt.zero(pipeline)  # moments and step count restart: the next step is a first step again
    g = synth.uniform(60, w0.shape, dt, 0.5, 2.0)
    memory.readFromBuffer(pipeline, layer.getGradients(lc)[0], g)
    before = download(pipeline, layer.getWeights()[0])
    opt.step(pipeline, cache)
    after = download(pipeline, layer.getWeights()[0])
    assert np.allclose(before.astype(np.float64) - after, lr, rtol=1e-3)
    opt.deinit(pipeline)
    cache.deinit(pipeline)
    layer.deinit(pipeline)


def test_layer_without_activation_mirrors_the_reference(env):
    # src/nn/layer/linear.zig:606-611 multiplies the sensitivity by a derivative tensor nothing fills
    context, pipeline = env
    layer = nn.Linear.init("f32", context, pipeline, 6, 4, None, seed=2)
    cache = nn.Cache.init(context, pipeline, 3, [layer])
    lc = cache.getLayerCache(0)
    x = upload(context, pipeline, "f32", synth.uniform(70, (3, 6), np.float32))
    y = upload(context, pipeline, "f32", synth.uniform(71, (3, 4), np.float32))
    assert np.array_equal(download(pipeline, layer.getSensitivity(lc)), np.ones((3, 4), np.float32))  # filled with one
    out = layer.forward(pipeline, x, lc)
    want = download(pipeline, x) @ download(pipeline, layer.getWeights()[0]).T
    assert np.allclose(download(pipeline, out), want, atol=1e-5)
    nn.loss.mse(True, pipeline, out, y, cache, None)
    layer.backward(pipeline, lc, x, None)
    assert not download(pipeline, layer.getGradients(lc)[0]).any()
    for t in (x, y):
        t.release(pipeline)
    cache.deinit(pipeline)
    layer.deinit(pipeline)


def test_xor_example_trains(env):
    """examples/xor_neural_network.zig: 2-10-1 sigmoid network, MSE, GD lr = 1.  The example runs 300
    iterations from clock-seeded weights; with a fixed seed 600 iterations reach the truth table."""
    context, pipeline = env
    inputs = upload(context, pipeline, "f32", np.array([[1, 1], [0, 1], [1, 0], [0, 0]], np.float32))
    expected_h = np.array([[0], [1], [1], [0]], np.float32)
    expected = upload(context, pipeline, "f32", expected_h)
    seq = nn.Sequential.init("f32")
    seq.append(nn.Linear.init("f32", context, pipeline, 2, 10, nn.Sigmoid.init(), seed=11))
    seq.append(nn.Linear.init("f32", context, pipeline, 10, 1, nn.Sigmoid.init(), seed=12))
    cache = nn.Cache.init(context, pipeline, 4, [seq])
    opt = nn.optimizers.GD.init("f32", 1.0)
    lc = cache.getLayerCache(0)
    layers = host_layers(pipeline, seq, [onn.SIGMOID, onn.SIGMOID], 1, np.float64)
    losses = []
    err = np.zeros(1, np.float32)
    for it in range(600):
        out = seq.forward(pipeline, inputs, lc)
        nn.loss.mse(True, pipeline, out, expected, cache, err if it % 100 == 0 else None)
        if it % 100 == 0:
            losses.append(float(err[0]))
        seq.backward(pipeline, lc, inputs, None)
        opt.step(pipeline, cache)
        if it < 50:  # the float64 restatement follows the same trajectory while rounding stays small
            onn.mlp_step(np.array([[1, 1], [0, 1], [1, 0], [0, 0]], np.float64), expected_h.astype(np.float64), layers, ("gd", 1.0))
            if it == 49:
                close(download(pipeline, seq.getWeights()[0]), layers[0]["w"][0], 10 * 50, "f32", "weights after 50 steps")
    final = download(pipeline, seq.forward(pipeline, inputs, lc))
    assert losses[-1] < 0.01 and losses[-1] < losses[0]
    assert np.array_equal(np.round(final), expected_h)
    opt.deinit(pipeline)
    cache.deinit(pipeline)
    seq.deinit(pipeline)
    inputs.release(pipeline)
    expected.release(pipeline)


def test_config5_mlp_training_step_full_size(env):
    """Benchmark configuration 5: 1024-4096-4096-1024, f32, batch 2048, tanh hidden / sigmoid output,
    MSE against uniform[0,1) targets, Adam lr = 1e-3, N(0,1) inputs, Xavier-uniform weights."""
    context, pipeline = env
    sizes, acts, batch = [1024, 4096, 4096, 1024], [onn.TANH, onn.TANH, onn.SIGMOID], 2048
    seq = build_network(context, pipeline, "f32", sizes, acts, seed=synth.config_seed(5, 0))
    layers = host_layers(pipeline, seq, acts, 1, np.float64)
    xh = synth.normal(synth.config_seed(5, 8), (batch, sizes[0]), np.float32)
    yh = synth.uniform(synth.config_seed(5, 9), (batch, sizes[-1]), np.float32, 0.0, 1.0)
    x, y = upload(context, pipeline, "f32", xh), upload(context, pipeline, "f32", yh)
    cache = nn.Cache.init(context, pipeline, batch, [seq])
    lc = cache.getLayerCache(0)
    opt = nn.optimizers.Adam.init("f32", 1e-3)
    w_before = [download(pipeline, w) for w in seq.getWeights()]
    out = seq.forward(pipeline, x, lc)
    loss = np.zeros(1, np.float32)
    nn.loss.mse(True, pipeline, out, y, cache, loss)
    seq.backward(pipeline, lc, x, None)
    opt.step(pipeline, cache)
    got_out = download(pipeline, out)
    got_g = [download(pipeline, g) for g in seq.getGradients(lc)]
    got_bg = [download(pipeline, g) for g in seq.getBiasGradients(lc)]
    got_w = [download(pipeline, w) for w in seq.getWeights()]

    eps = float(np.finfo(np.float32).eps)
    want_out, want_err, want_grads, _ = onn.mlp_step(xh.astype(np.float64), yh.astype(np.float64), layers,
                                                     ("adam", 1e-3, 0.9, 0.999, eps))
    close(got_out, want_out, 4096 * 3, "f32", "output")
    assert abs(float(loss[0]) - want_err.mean()) <= 1e-5 * np.sqrt(4096 * 3)
    for i in range(3):
        close(got_g[i], want_grads[i][0][0], 4096 * 3 * batch, "f32", f"gradient {i}")
        close(got_bg[i], want_grads[i][1][0], 4096 * 3 * batch, "f32", f"bias gradient {i}")
        # first Adam step moves every weight by lr * g / (|g| + eps): compare where |g| is well above
        # the rounding of g itself, elsewhere only bound the move
        step = got_w[i].astype(np.float64) - w_before[i]
        assert np.abs(step).max() <= 1e-3 * (1 + 1e-3)
        g = want_grads[i][0][0]
        firm = np.abs(g) > 1e-3 * np.abs(g).max()
        want_step = layers[i]["w"][0] - w_before[i].astype(np.float64)
        assert np.allclose(step[firm], want_step[firm], rtol=0, atol=1e-3 * 0.02 + 4 * eps * np.abs(w_before[i]).max())
    opt.deinit(pipeline)
    cache.deinit(pipeline)
    seq.deinit(pipeline)
    x.release(pipeline)
    y.release(pipeline)


# ---- the fused passes against the separate ones (raw C ABI) ---------------------------------------

@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("rows,cols,pad", [(1, 1, 0), (5, 3, 0), (19, 11, 1), (64, 256, 0), (33, 65, 3), (300, 1000, 8),
                                           (2048, 1024, 128), (1000, 4100, 4)])
def test_sensitivity_step_equals_the_three_passes(dev, dtype, rows, cols, pad):
    """wk_sensitivity_step = wk_activation_dev + wk_hadamard + wk_bias_step, bit for bit (same
    arithmetic per element, same order of additions per column), for sigmoid, tanh and no activation,
    aligned and unaligned pitches, with and without a bias gradient; gaps between rows keep their
    poison.  The separate passes are in turn held to the restatement by the tests above."""
    import ctypes
    from wekua_amd import raw
    dt = NP[dtype]
    did = raw.dtype_id(dtype)
    lib = dev.lib
    pitch = cols + pad
    s3 = (ctypes.c_uint64 * 3)(1, rows, cols)

    def padded(host, poison):
        full = np.full((rows, pitch), poison, dtype=dt)
        full[:, :cols] = host
        return full

    out_h = synth.uniform(61, (rows, cols), dt, 0.05, 0.95)     # a sigmoid / tanh output
    sens_h = synth.uniform(62, (rows, cols), dt, -2.0, 2.0)
    dev_h = synth.uniform(63, (rows, cols), dt, -1.0, 1.0)      # what a layer without activation multiplies by
    for kind in (0, 1, -1):
        for with_bias in (True, False):
            # separate passes
            d_out = dev.upload(padded(out_h, 7))
            d_sens = dev.upload(padded(sens_h, 8))
            d_dev = dev.upload(padded(dev_h, 9))
            d_bg = dev.upload(np.full(cols + 4, -3, dtype=dt))
            if kind >= 0:
                assert lib.wk_activation_dev(dev.stream, did, kind, s3, d_out.ptr, pitch, 0, d_dev.ptr, pitch, 0) == 0
            assert lib.wk_hadamard(dev.stream, did, s3, d_sens.ptr, pitch, 0, d_dev.ptr, pitch, 0) == 0
            if with_bias:
                assert lib.wk_bias_step(dev.stream, did, rows, cols, d_sens.ptr, pitch, d_bg.ptr) == 0
            dev.sync()
            want = [d.download(dt, (rows, pitch)) for d in (d_sens, d_dev, d_out)] + [d_bg.download(dt, (cols + 4,))]
            for d in (d_out, d_sens, d_dev, d_bg):
                d.free()
            # one pass
            f_out = dev.upload(padded(out_h, 7))
            f_sens = dev.upload(padded(sens_h, 8))
            f_dev = dev.upload(padded(dev_h, 9))
            f_bg = dev.upload(np.full(cols + 4, -3, dtype=dt))
            assert lib.wk_sensitivity_step(dev.stream, did, kind, rows, cols, f_out.ptr if kind >= 0 else None, pitch, f_sens.ptr, pitch,
                                           f_dev.ptr, pitch, f_bg.ptr if with_bias else None) == 0
            dev.sync()
            got = [d.download(dt, (rows, pitch)) for d in (f_sens, f_dev, f_out)] + [f_bg.download(dt, (cols + 4,))]
            for d in (f_out, f_sens, f_dev, f_bg):
                d.free()
            for name, g, w in zip(("sensitivity", "derivative", "output", "bias gradient"), got, want):
                assert np.array_equal(g, w), f"{name} kind={kind} bias={with_bias} {rows}x{cols}+{pad}"
            assert np.array_equal(got[2][:, :cols], out_h)     # the layer's output is read only
    buf = dev.malloc(4096)
    p = buf.ptr
    assert lib.wk_sensitivity_step(dev.stream, did, 2, 4, 4, p, 4, p, 4, p, 4, None) == 1       # unknown activation
    assert lib.wk_sensitivity_step(dev.stream, did, 0, 4, 4, None, 4, p, 4, p, 4, None) == 1    # sigmoid needs the output
    assert lib.wk_sensitivity_step(dev.stream, did, 0, 4, 8, p, 8, p, 4, p, 8, None) == 1       # pitch < cols
    assert lib.wk_sensitivity_step(dev.stream, raw.dtype_id("i32"), 0, 4, 4, p, 4, p, 4, p, 4, None) == 9
    buf.free()


@pytest.mark.parametrize("dtype", ["f32", "f64"])
def test_adam_step_multi_equals_one_launch_per_tensor(dev, dtype):
    """wk_adam_step_multi over a list of parameter tensors (more than one launch's worth, ragged
    widths, pitched rows) against wk_adam_step on copies of the same tensors: the same bits in the
    weights and both moments after three steps; an unaligned tensor in the list takes the per-tensor
    route and still agrees."""
    import ctypes
    from wekua_amd import raw
    from wekua_amd._capi import WkAdamTensor
    dt = NP[dtype]
    did = raw.dtype_id(dtype)
    lib = dev.lib
    for shapes in ([(1, 1, 5, 5), (1, 64, 256, 256), (1, 33, 65, 68), (2, 7, 12, 12), (1, 1, 4096, 4096), (1, 300, 1000, 1000),
                    (1, 1, 1, 4), (1, 128, 512, 520), (1, 17, 130, 132), (1, 1, 70, 72)],
                   [(1, 19, 11, 13), (1, 64, 64, 64)]):                       # (depth, rows, cols, pitch); 13 is not 16-byte aligned
        sets = []
        for which in range(2):
            bufs = []
            for i, (d, r, c, p) in enumerate(shapes):
                arrs = [synth.uniform(100 + 4 * i + j, (d, r, p), dt, 0.0 if j == 3 else -1.0, 1.0) for j in range(4)]
                bufs.append([dev.upload(a) for a in arrs])                        # w, g, m, v (v >= 0)
            sets.append(bufs)
        lr, b1, b2, eps = 1e-3, 0.9, 0.999, float(np.finfo(dt).eps)
        for step in (1, 2, 3):
            for (d, r, c, p), (w, g, m, v) in zip(shapes, sets[0]):
                s3 = (ctypes.c_uint64 * 3)(d, r, c)
                assert lib.wk_adam_step(dev.stream, did, s3, w.ptr, p, r * p, g.ptr, p, r * p, m.ptr, v.ptr, p, r * p, lr, b1, b2, eps, step) == 0
            lst = (WkAdamTensor * len(shapes))()
            for t, (d, r, c, p), (w, g, m, v) in zip(lst, shapes, sets[1]):
                t.w, t.g, t.m, t.v = w.ptr.value, g.ptr.value, m.ptr.value, v.ptr.value
                t.shape3[0], t.shape3[1], t.shape3[2] = d, r, c
                t.w_row_pitch = t.g_row_pitch = t.mv_row_pitch = p
                t.w_slice_pitch = t.g_slice_pitch = t.mv_slice_pitch = r * p
            assert lib.wk_adam_step_multi(dev.stream, did, len(shapes), lst, lr, b1, b2, eps, step) == 0
        dev.sync()
        for (d, r, c, p), one, many in zip(shapes, sets[0], sets[1]):
            for name, a, b in zip("wgmv", one, many):
                assert np.array_equal(a.download(dt, (d, r, p)), b.download(dt, (d, r, p))), f"{name} of {(d, r, c, p)}"
        for bufs in sets:
            for quad in bufs:
                for b in quad:
                    b.free()
    assert lib.wk_adam_step_multi(dev.stream, did, 0, None, 1e-3, 0.9, 0.999, 1e-8, 1) == 0
    assert lib.wk_adam_step_multi(dev.stream, did, 1, None, 1e-3, 0.9, 0.999, 1e-8, 1) == 1
