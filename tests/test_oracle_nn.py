"""CPU: pins the numpy restatement of the nn kernels and of the MLP training step (oracle/nn.py)
against the reference's own known answers where it holds any, and against mathematics elsewhere
(central differences, closed forms, brute force on tiny inputs)."""
import numpy as np
import pytest

from oracle import nn as onn

FLOATS = [np.float32, np.float64]


# ---- the reference's own known answers -----------------------------------------------------------

@pytest.mark.parametrize("dt", FLOATS)
def test_dot_known_answer(dt):
    # src/math/basic.zig:258-320: [1,2,3,4] * [2,3,4,5] = [2,6,12,20]
    x = np.arange(1, 5, dtype=dt)
    y = np.arange(2, 6, dtype=dt)
    assert np.array_equal(onn.hadamard(x, y), np.array([2, 6, 12, 20], dtype=dt))


@pytest.mark.parametrize("dt", FLOATS)
def test_sum_and_mean_known_answers(dt):
    # src/math/basic.zig:322-366: sum [1..5] = 15;  :368-420: mean [2,4,6,8] = 5
    assert onn.tensor_sum(np.arange(1, 6, dtype=dt)) == dt(15)
    assert abs(float(onn.tensor_mean(np.array([2, 4, 6, 8], dtype=dt))) - 5.0) < 1e-5


@pytest.mark.parametrize("dt", FLOATS)
def test_tanh_known_answer(dt):
    # src/math/trig.zig:397-450: tanh(0) = 0, tanh(1) ~ 0.7616 within 1e-4
    got = onn.activation(onn.TANH, np.array([0, 1], dtype=dt))
    assert abs(float(got[0])) < 1e-4 and abs(float(got[1]) - 0.7616) < 1e-4


# ---- mathematics ---------------------------------------------------------------------------------

def test_sum_matches_exact_rational_sum():
    rng = np.random.default_rng(1)
    x = rng.integers(-1000, 1000, size=(7, 13)).astype(np.float64)  # exactly representable
    assert onn.tensor_sum(x) == float(sum(int(v) for v in x.ravel()))
    assert onn.tensor_mean(x) == onn.tensor_sum(x) / x.size


def test_sigmoid_special_values_and_symmetry():
    x = np.array([-30.0, -2.0, 0.0, 2.0, 30.0])
    y = onn.activation(onn.SIGMOID, x)
    assert y[2] == 0.5
    assert np.allclose(y + y[::-1], 1.0, atol=1e-15)  # s(x) + s(-x) = 1
    assert np.allclose(y[3], 1.0 / (1.0 + np.exp(-2.0)))
    assert np.allclose(np.log(y[3] / (1 - y[3])), 2.0)  # logit inverts it


@pytest.mark.parametrize("kind", [onn.SIGMOID, onn.TANH])
def test_activation_derivative_against_central_differences(kind):
    x = np.linspace(-3, 3, 41)
    h = 1e-6
    numeric = (onn.activation(kind, x + h) - onn.activation(kind, x - h)) / (2 * h)
    assert np.allclose(onn.activation_dev(kind, onn.activation(kind, x)), numeric, atol=1e-9)


def test_bias_and_bias_step_brute_force():
    rng = np.random.default_rng(2)
    out = rng.standard_normal((5, 3))
    bias = rng.standard_normal(3)
    got = onn.bias_add(out, bias)
    for r in range(5):
        for c in range(3):
            assert got[r, c] == out[r, c] + bias[c]
    ints = rng.integers(-50, 50, size=(6, 4)).astype(np.float64)
    assert np.array_equal(onn.bias_step(ints), np.array([sum(ints[:, c]) for c in range(4)]))


def test_mse_brute_force():
    out = np.array([[0.25, 1.0], [2.0, -1.0]])
    exp = np.array([[1.0, 1.0], [0.0, 0.5]])
    err, dev = onn.mse(out, exp)
    assert np.array_equal(err, np.array([[0.5625, 0.0], [4.0, 2.25]]))
    assert np.array_equal(dev, np.array([[-1.5, 0.0], [4.0, -3.0]]))  # d/d out of (exp - out)^2


def _random_layers(rng, sizes, acts, deep=1, bias=True):
    layers = []
    for (i, o), act in zip(zip(sizes[:-1], sizes[1:]), acts):
        w = [rng.uniform(-0.7, 0.7, size=(o, i if d == 0 else o)) for d in range(deep)]
        b = [rng.uniform(-0.3, 0.3, size=o) if bias else None for _ in range(deep)]
        layers.append({"w": w, "b": b, "act": act})
    return layers


def _loss(x, expected, layers):
    out = onn.mlp_forward(x, layers)[-1][-1]
    return float(np.sum((expected - out) ** 2))


@pytest.mark.parametrize("deep", [1, 2])
def test_network_gradients_against_central_differences(deep):
    """The reference's loss derivative is -2(expected - output) without a 1/N factor, so backward
    yields the gradient of the SUM of squared errors."""
    rng = np.random.default_rng(3)
    sizes, acts = [3, 5, 4, 2], [onn.TANH, onn.SIGMOID, onn.TANH]
    layers = _random_layers(rng, sizes, acts, deep=deep)
    x = rng.standard_normal((6, 3))
    expected = rng.uniform(-1, 1, size=(6, 2))
    caches = onn.mlp_forward(x, layers)
    _, sens = onn.mse(caches[-1][-1], expected)
    grads = onn.mlp_backward(x, layers, caches, sens)
    h = 1e-6
    for li, layer in enumerate(layers):
        for d in range(deep):
            for kind, params, got in (("w", layer["w"], grads[li][0]), ("b", layer["b"], grads[li][1])):
                p = params[d]
                numeric = np.zeros_like(p)
                it = np.nditer(p, flags=["multi_index"])
                for _ in it:
                    idx = it.multi_index
                    keep = p[idx]
                    p[idx] = keep + h
                    up = _loss(x, expected, layers)
                    p[idx] = keep - h
                    down = _loss(x, expected, layers)
                    p[idx] = keep
                    numeric[idx] = (up - down) / (2 * h)
                assert np.allclose(got[d], numeric, rtol=1e-6, atol=1e-8), (li, d, kind)


def test_layer_without_activation_gets_zero_gradients():
    # linear.zig:606-611: the sensitivity is multiplied by the derivative tensor, which nothing fills
    rng = np.random.default_rng(4)
    layers = _random_layers(rng, [3, 2], [None])
    x = rng.standard_normal((4, 3))
    caches = onn.mlp_forward(x, layers)
    _, sens = onn.mse(caches[-1][-1], np.zeros((4, 2)))
    g, bg = onn.mlp_backward(x, layers, caches, sens)[0]
    assert not g[0].any() and not bg[0].any()


def test_gd_step_reduces_the_loss_and_equals_axpy():
    rng = np.random.default_rng(5)
    layers = _random_layers(rng, [2, 10, 1], [onn.SIGMOID, onn.SIGMOID])
    x = np.array([[1, 1], [0, 1], [1, 0], [0, 0]], dtype=np.float64)
    y = np.array([[0], [1], [1], [0]], dtype=np.float64)
    before = _loss(x, y, layers)
    w0 = layers[0]["w"][0].copy()
    _, _, grads, _ = onn.mlp_step(x, y, layers, ("gd", 0.1))
    assert np.array_equal(layers[0]["w"][0], w0 + (-0.1) * grads[0][0][0])
    assert _loss(x, y, layers) < before
    for _ in range(3000):  # examples/xor_neural_network.zig trains this network with GD
        onn.mlp_step(x, y, layers, ("gd", 1.0))
    assert _loss(x, y, layers) < 0.05


@pytest.mark.parametrize("dt", FLOATS)
def test_adam_first_step_closed_form(dt):
    # m0 = v0 = 0: m_hat = g, v_hat = g^2, so dw = -lr * g / (|g| + eps)
    g = np.array([0.5, -2.0, 1e-3, 3.0], dtype=dt)
    w = np.ones(4, dtype=dt)
    lr, eps = 1e-3, 1e-8
    w1, m, v = onn.adam_update(w, g, np.zeros(4, dt), np.zeros(4, dt), lr, 0.9, 0.999, eps, 1)
    want = 1.0 - lr * g.astype(np.float64) / (np.abs(g.astype(np.float64)) + eps)
    assert np.allclose(w1, want, rtol=4 * np.finfo(dt).eps)
    assert np.allclose(m, 0.1 * g, rtol=1e-6) and np.allclose(v, 0.001 * g * g, rtol=1e-5)


def test_adam_converges_on_a_quadratic():
    w = np.array([5.0, -3.0])
    m = v = np.zeros(2)
    for t in range(1, 4001):
        w, m, v = onn.adam_update(w, 2 * w, m, v, 1e-2, 0.9, 0.999, 1e-8, t)
    assert np.all(np.abs(w) < 1e-3)


@pytest.mark.parametrize("dt", FLOATS)
@pytest.mark.parametrize("eps_kind", ["machine", "1e-8"])
def test_adam_matches_the_library_routine_over_several_steps(dt, eps_kind):
    """The reference has no Adam (src/nn/optimizers/adam.zig is empty), so the pin is the library
    routine of the same rule: torch.optim.Adam on CPU tensors, epsilon added outside the
    bias-corrected root.  Nine steps with fresh random gradients: a wrong exponent in a bias
    correction, swapped betas or epsilon inside the root all show from step two on."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(17)
    n = 257
    lr, b1, b2 = 1e-3, 0.9, 0.999
    eps = float(np.finfo(dt).eps) if eps_kind == "machine" else 1e-8
    w = rng.standard_normal(n).astype(dt)
    m = np.zeros(n, dt)
    v = np.zeros(n, dt)
    p = torch.tensor(w.copy(), requires_grad=True)
    opt = torch.optim.Adam([p], lr=lr, betas=(b1, b2), eps=eps, foreach=False, fused=False)
    m_scale = np.zeros(n)
    for t in range(1, 10):
        g = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 2, n)).astype(dt)
        w, m, v = onn.adam_update(w, g, m, v, lr, b1, b2, eps, t)
        m_scale = b1 * m_scale + (1 - b1) * np.abs(g)      # what the sum for m is rounded against
        p.grad = torch.tensor(g.copy())
        opt.step()
        st = opt.state[p]
        assert w.dtype == dt
        # one unit in the last place of the weight per step taken (two rounded trajectories; a
        # wrong rule moves a weight by about lr = 1e-3 per step); the moments to a few roundings
        assert np.all(np.abs(p.detach().numpy() - w) <= t * np.spacing(np.abs(w).astype(dt))), t
        assert np.all(np.abs(st["exp_avg"].numpy() - m) <= 8 * np.finfo(dt).eps * m_scale), t
        assert np.allclose(st["exp_avg_sq"].numpy(), v, rtol=8 * np.finfo(dt).eps, atol=1e-30), t


def test_adam_pin_sees_a_wrong_bias_correction():
    """The comparison above is sharp enough to catch the mistakes it is there for."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(3)
    n = 64
    w0 = rng.standard_normal(n)
    gs = [rng.standard_normal(n) for _ in range(5)]
    p = torch.tensor(w0.copy(), requires_grad=True)
    opt = torch.optim.Adam([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, foreach=False, fused=False)
    for g in gs:
        p.grad = torch.tensor(g.copy())
        opt.step()
    want = p.detach().numpy()

    def run(b1, b2, tshift):
        w, m, v = w0.copy(), np.zeros(n), np.zeros(n)
        for t, g in enumerate(gs, 1):
            w, m, v = onn.adam_update(w, g, m, v, 1e-3, b1, b2, 1e-8, max(1, t + tshift))
        return w

    assert np.abs(run(0.9, 0.999, 0) - want).max() <= 1e-15
    assert np.abs(run(0.999, 0.9, 0) - want).max() > 1e-5      # swapped betas
    assert np.abs(run(0.9, 0.999, -1) - want).max() > 1e-5     # bias correction one step behind
