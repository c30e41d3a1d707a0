"""CPU restatement (numpy) of the reference's neural-network kernels and of one MLP training step.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of the benchmarks -- never by the product path, which runs on the GPU or fails.

Every function works on the LOGICAL elements in the dtype it is given (np.float32 / np.float64);
passing float64 turns the whole step into the semantic reference the f32 device results are
compared with.

Pin status
----------
* hadamard, sum, mean, tanh: checked against the reference's own known answers
  (src/math/basic.zig:258-420, src/math/trig.zig:397-450) in tests/test_oracle_nn.py.
* sigmoid / sigmoid_dev / tanh_dev, mse, bias_add, bias_step, linear_forward, linear_backward,
  mlp_step (forward + backward): the reference holds no known answers; pinned by mathematics --
  the derivative kernels against central differences of the activations, and the gradients of the
  whole network against central differences of sum((expected - output)^2) in float64, which fails
  for a dropped term, a wrong sign, a transposed operand or a wrong layer index.
* gd_update: equals blas.axpy with alpha = -lr, which is pinned by the reference's axpy table.
* adam_update: PARITY UNPINNED.  The reference's Zig tree has no Adam (src/nn/optimizers/adam.zig
  is empty), so there is nothing of the reference to match; the textbook rule is restated and
  checked only against its closed form for the first step (|dw| = lr * |g| / (|g| + eps)).

Known layout-dependent behaviour of the reference that is NOT restated: its element-wise kernels
also run over the padding columns of its padded tensors (sigmoid turns padding zeros into 0.5,
which math.mean then counts in loss.mse's error_result when the last dimension is padded).  The
logical elements, which is all this module and the device path define, are unaffected.
"""
from __future__ import annotations

import numpy as np

SIGMOID, TANH = 0, 1


def hadamard(x, y):
    """math.dot (src/math/kernels/dot.cl): x * y element-wise."""
    return x * y


def tensor_sum(x):
    """math.sum (src/math/kernels/sum.cl:30-41 then src/math/basic.zig:186-199): every row is summed
    left to right on the device, the row sums are then added in order on the host."""
    x2 = x.reshape(-1, x.shape[-1])
    rows = np.zeros(x2.shape[0], dtype=x.dtype)
    for k in range(x2.shape[1]):
        rows = rows + x2[:, k]
    total = x.dtype.type(0)
    for v in rows:
        total = x.dtype.type(total + v)
    return total


def tensor_mean(x):
    """math.mean (src/math/basic.zig:203-244): sum / number_of_elements_without_padding."""
    return x.dtype.type(tensor_sum(x) / x.dtype.type(x.size))


def activation(kind: int, x):
    """Sigmoid 1/(1+exp(-x)) (src/nn/activation/kernels/sigmoid.cl:15-16);
    Tanh tanh(x) (src/math/kernels/trig.cl:65)."""
    one = x.dtype.type(1)
    if kind == SIGMOID:
        return (one / (one + np.exp(-x))).astype(x.dtype)
    if kind == TANH:
        return np.tanh(x).astype(x.dtype)
    raise ValueError(kind)


def activation_dev(kind: int, y):
    """Derivative from the activation OUTPUT y: y(1-y) (sigmoid.cl:35-36); 1 - y*y (tanh.cl:17-18)."""
    one = y.dtype.type(1)
    if kind == SIGMOID:
        return y * (one - y)
    if kind == TANH:
        return one - y * y
    raise ValueError(kind)


def bias_add(out, bias):
    """src/nn/layer/kernels/bias.cl:17: out[r][c] += bias[c]."""
    return out + bias[None, :]


def bias_step(sens):
    """src/nn/layer/kernels/bias_step.cl:30-37: column sums, rows added top to bottom."""
    res = np.zeros(sens.shape[1], dtype=sens.dtype)
    for r in range(sens.shape[0]):
        res = res + sens[r]
    return res


def mse(output, expected):
    """src/nn/loss/kernels/mse.cl:27-31: err = expected - output; returns (err*err, -2*err)."""
    err = expected - output
    return err * err, output.dtype.type(-2) * err


def matmul(a, op_a, b, op_b):
    """blas.gemm with alpha = beta = null in the dtype of the operands (K accumulated by numpy)."""
    return (a.T if op_a else a) @ (b.T if op_b else b)


def linear_forward(x, weights, biases, kind):
    """Linear.forward (src/nn/layer/linear.zig:480-525) for the `deep` list of matrices of one
    layer: out = in * W^T, += bias, activation.  Returns the list of cached outputs."""
    outs = []
    for w, b in zip(weights, biases):
        o = matmul(x, 0, w, 1)
        if b is not None:
            o = bias_add(o, b)
        if kind is not None:
            o = activation(kind, o)
        outs.append(o)
        x = o
    return outs


def linear_backward(x, weights, outs, sens_last, kind, has_bias=True, want_input_sens=True):
    """Linear.backward (linear.zig:579-678).  `sens_last` is the sensitivity of the layer's last
    output.  Returns (gradients, bias_gradients, input_sensitivity)."""
    n = len(weights)
    grads, bgrads = [None] * n, [None] * n
    sens = sens_last
    for i in range(n - 1, -1, -1):
        # without an activation the reference multiplies by the zero-filled derivative tensor
        dev = activation_dev(kind, outs[i]) if kind is not None else np.zeros_like(outs[i])
        sens = hadamard(sens, dev)
        prev = outs[i - 1] if i >= 1 else x
        grads[i] = matmul(sens, 1, prev, 0)
        if has_bias:
            bgrads[i] = bias_step(sens)
        if i == 0 and not want_input_sens:
            return grads, bgrads, None
        sens = matmul(sens, 0, weights[i], 0)
    return grads, bgrads, sens


def mlp_forward(x, layers):
    """Sequential.forward (src/nn/layer/sequential.zig:210-226).  layers: list of dicts with keys
    w (list), b (list of arrays or None), act (SIGMOID / TANH / None)."""
    caches = []
    for l in layers:
        outs = linear_forward(x, l["w"], l["b"], l["act"])
        caches.append(outs)
        x = outs[-1]
    return caches


def mlp_backward(x, layers, caches, sens_last):
    """Sequential.backward (sequential.zig:242-274): last layer to first."""
    grads = [None] * len(layers)
    sens = sens_last
    for i in range(len(layers) - 1, -1, -1):
        inp = caches[i - 1][-1] if i >= 1 else x
        has_bias = layers[i]["b"][0] is not None
        g, bg, sens = linear_backward(inp, layers[i]["w"], caches[i], sens, layers[i]["act"], has_bias,
                                      want_input_sens=i >= 1)
        grads[i] = (g, bg)
    return grads


def gd_update(w, g, lr):
    """GD.step (src/nn/optimizers/gd.zig:39,62-71): blas.axpy(g, -lr, w)."""
    return w + w.dtype.type(-lr) * g


def adam_update(w, g, m, v, lr, beta1, beta2, eps, t):
    """Textbook Adam (no reference counterpart): returns (w, m, v) after step t (1-based).  The
    bias corrections are formed in float64 on the host and rounded to the element type once."""
    T = w.dtype.type
    b1, b2, ib1, ib2 = T(beta1), T(beta2), T(1.0 - beta1), T(1.0 - beta2)
    m = b1 * m + ib1 * g
    v = b2 * v + (ib2 * g) * g
    step_size = T(lr / (1.0 - beta1 ** t))
    inv_sqrt_c2 = T(1.0 / np.sqrt(1.0 - beta2 ** t))
    w = w - step_size * m / (np.sqrt(v) * inv_sqrt_c2 + T(eps))
    return w.astype(w.dtype), m, v


def mlp_step(x, expected, layers, optimizer, state=None):
    """One training step as examples/xor_neural_network.zig:117-127 drives it: forward, loss.mse with
    derivative, backward, optimizer step.  `optimizer`: ("gd", lr) or ("adam", lr, b1, b2, eps).
    Updates `layers` in place; returns (output, error_tensor, gradients, state)."""
    caches = mlp_forward(x, layers)
    out = caches[-1][-1]
    err, sens = mse(out, expected)
    grads = mlp_backward(x, layers, caches, sens)
    if optimizer[0] == "gd":
        for l, (g, bg) in zip(layers, grads):
            l["w"] = [gd_update(w, gi, optimizer[1]) for w, gi in zip(l["w"], g)]
            l["b"] = [gd_update(b, bgi, optimizer[1]) if b is not None else None for b, bgi in zip(l["b"], bg)]
    elif optimizer[0] == "adam":
        _, lr, b1, b2, eps = optimizer
        if state is None:
            state = {"t": 0, "mv": {}}
        state["t"] += 1
        for li, (l, (g, bg)) in enumerate(zip(layers, grads)):
            for kind, params, gr in (("w", l["w"], g), ("b", l["b"], bg)):
                for i, (p, gi) in enumerate(zip(params, gr)):
                    if p is None:
                        continue
                    key = (li, kind, i)
                    m, v = state["mv"].get(key, (np.zeros_like(p), np.zeros_like(p)))
                    p2, m, v = adam_update(p, gi, m, v, lr, b1, b2, eps, state["t"])
                    state["mv"][key] = (m, v)
                    params[i] = p2
    else:
        raise ValueError(optimizer)
    return out, err, grads, state
