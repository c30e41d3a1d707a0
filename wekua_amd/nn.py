"""wekua_amd.nn -- Python binding of the host mirror of wekua's `nn` and `math` modules
(wekua_amd/host/wekua_nn.hpp), with the reference's names and call order, so that a training loop
reads like examples/xor_neural_network.zig:

    seq = nn.Sequential.init("f32")
    seq.append(nn.Linear.init("f32", ctx, pipeline, 2, 10, nn.Sigmoid.init()))
    seq.append(nn.Linear.init("f32", ctx, pipeline, 10, 1, nn.Sigmoid.init()))
    cache = nn.Cache.init(ctx, pipeline, 4, [seq])
    opt = nn.optimizers.GD.init("f32", lr=1.0)
    layer_cache = cache.getLayerCache(0)
    for _ in range(300):
        out = seq.forward(pipeline, inputs, layer_cache)
        nn.loss.mse(True, pipeline, out, expected, cache, None)
        seq.backward(pipeline, layer_cache, inputs, None)
        opt.step(pipeline, cache)

f32 and f64 only, like the reference's nn module.  Everything runs on the device through
libwekua_hip.so; there is no host fallback.
"""
from __future__ import annotations

import ctypes
import enum

import numpy as np

import wekua_amd as _w
from .raw import dtype_id, real_np_dtype

vp, u64 = ctypes.c_void_p, ctypes.c_uint64


class ActivationKind(enum.IntEnum):
    none = -1
    sigmoid = 0
    tanh = 1


class Activation:
    """nn.activation.Activation (src/nn/activation/main.zig)."""

    def __init__(self, kind: ActivationKind):
        self.kind = ActivationKind(kind)

    def run(self, pipeline, net_output) -> None:
        _w._check(_w._lib().wkz_nn_activation_run(int(self.kind), pipeline._h, net_output._h), "Activation.run")

    def getDerivative(self, pipeline, output, derivative) -> None:
        _w._check(_w._lib().wkz_nn_activation_get_derivative(int(self.kind), pipeline._h, output._h, derivative._h),
                  "Activation.getDerivative")


class Sigmoid:
    @staticmethod
    def init() -> Activation:
        return Activation(ActivationKind.sigmoid)


class Tanh:
    @staticmethod
    def init() -> Activation:
        return Activation(ActivationKind.tanh)


class Layer:
    """nn.layer.Layer (src/nn/layer/main.zig): the interface Linear and Sequential share."""

    def __init__(self, handle, dtype: str, context):
        self._h = handle
        self.dtype = dtype
        self.context = context

    def deinit(self, pipeline) -> None:
        if self._h:
            _w._check(_w._lib().wkz_nn_layer_deinit(self._h, pipeline._h), "Layer.deinit")
            self._h = None

    def _tensors(self, which: int, layer_cache):
        lib = _w._lib()
        count = u64()
        _w._check(lib.wkz_nn_layer_tensor(self._h, layer_cache, which, 0, ctypes.byref(count), None), "Layer tensors")
        out = []
        for i in range(count.value):
            h = vp()
            _w._check(lib.wkz_nn_layer_tensor(self._h, layer_cache, which, i, None, ctypes.byref(h)), "Layer tensors")
            out.append(_w.Tensor._borrow(h, self.dtype, self.context) if h else None)
        return out

    def getWeights(self):
        return self._tensors(0, None)

    def getBias(self):
        return self._tensors(1, None)

    def getGradients(self, layer_cache):
        return self._tensors(2, layer_cache)

    def getBiasGradients(self, layer_cache):
        return self._tensors(3, layer_cache)

    def getCachedOutput(self, layer_cache):
        return self._tensors(4, layer_cache)[0]

    def getSensitivity(self, layer_cache):
        return self._tensors(5, layer_cache)[0]

    def forward(self, pipeline, input_tensor, layer_cache):
        h = vp()
        _w._check(_w._lib().wkz_nn_layer_forward(self._h, pipeline._h, input_tensor._h, layer_cache, ctypes.byref(h)),
                  "Layer.forward")
        return _w.Tensor._borrow(h, self.dtype, self.context)

    def backward(self, pipeline, layer_cache, input_tensor, input_gradient=None) -> None:
        _w._check(_w._lib().wkz_nn_layer_backward(self._h, pipeline._h, layer_cache, input_tensor._h,
                                                  input_gradient._h if input_gradient is not None else None),
                  "Layer.backward")


class Linear(Layer):
    """nn.layer.Linear (src/nn/layer/linear.zig)."""

    @classmethod
    def init(cls, dtype: str, context, pipeline, input: int, output: int, acti: "Activation | None" = None,
             deep: int = 1, enable_bias: bool = True, seed: "int | None" = None) -> "Linear":
        h = vp()
        seed_arg = ctypes.byref(u64(seed)) if seed is not None else None
        _w._check(_w._lib().wkz_nn_linear_init(context._h, pipeline._h, dtype_id(dtype), input, output,
                                               int(acti.kind) if acti is not None else -1, deep, int(enable_bias),
                                               seed_arg, ctypes.byref(h)), "Linear.init")
        return cls(h, dtype, context)


class Sequential(Layer):
    """nn.layer.Sequential (src/nn/layer/sequential.zig): owns the layers appended to it."""

    @classmethod
    def init(cls, dtype: str, context=None) -> "Sequential":
        h = vp()
        _w._check(_w._lib().wkz_nn_sequential_init(dtype_id(dtype), ctypes.byref(h)), "Sequential.init")
        return cls(h, dtype, context)

    def append(self, layer: Layer) -> None:
        if self.context is None:
            self.context = layer.context
        _w._check(_w._lib().wkz_nn_sequential_append(self._h, layer._h), "Sequential.append")
        layer._h = None  # owned by the sequence from here on


class Cache:
    """nn.layer.Cache (src/nn/layer/cache.zig): per-batch-size state of a list of layers."""

    def __init__(self, handle, dtype: str, context):
        self._h = handle
        self.dtype = dtype
        self.context = context

    @classmethod
    def init(cls, context, pipeline, number_of_elements: int, layers) -> "Cache":
        arr = (vp * len(layers))(*[l._h for l in layers])
        h = vp()
        _w._check(_w._lib().wkz_nn_cache_init(context._h, pipeline._h, number_of_elements, arr, len(layers), ctypes.byref(h)),
                  "Cache.init")
        return cls(h, layers[0].dtype, context)

    def getLayerCache(self, index: int):
        p = _w._lib().wkz_nn_cache_get_layer_cache(self._h, index)
        if not p:
            raise IndexError(index)
        return vp(p)

    @property
    def error_tensor(self):
        h = vp()
        _w._check(_w._lib().wkz_nn_cache_error_tensor(self._h, ctypes.byref(h)), "Cache.error_tensor")
        return _w.Tensor._borrow(h, self.dtype, self.context)

    def deinit(self, pipeline) -> None:
        if self._h:
            _w._check(_w._lib().wkz_nn_cache_deinit(self._h, pipeline._h), "Cache.deinit")
            self._h = None


class loss:
    @staticmethod
    def mse(calculate_derivative: bool, pipeline, output, expected, cache: Cache, error_result: "np.ndarray | None"):
        """loss.mse (src/nn/loss/mse.zig:63-132).  `error_result`: a one-element array that receives
        the mean squared error (this drains the pipeline), or None."""
        ptr = None
        if error_result is not None:
            if error_result.dtype != real_np_dtype(cache.dtype) or error_result.size != 1:
                raise TypeError("error_result must be a one-element array of the tensors' dtype")
            ptr = error_result.ctypes.data
        _w._check(_w._lib().wkz_nn_loss_mse(int(calculate_derivative), pipeline._h, output._h, expected._h, cache._h, ptr),
                  "loss.mse")


class Optimizer:
    """nn.optimizers.Optimizer (src/nn/optimizers/main.zig)."""

    def __init__(self, handle, dtype):
        self._h = handle
        self.dtype = dtype

    def step(self, pipeline, cache: Cache) -> None:
        _w._check(_w._lib().wkz_nn_optimizer_step(self._h, pipeline._h, cache._h), "Optimizer.step")

    def zero(self, pipeline) -> None:
        _w._check(_w._lib().wkz_nn_optimizer_zero(self._h, pipeline._h), "Optimizer.zero")

    def deinit(self, pipeline) -> None:
        if self._h:
            _w._check(_w._lib().wkz_nn_optimizer_deinit(self._h, pipeline._h), "Optimizer.deinit")
            self._h = None


class optimizers:
    class GD:
        """Gradient descent (src/nn/optimizers/gd.zig): w += (-lr) * g through blas.axpy."""

        @staticmethod
        def init(dtype: str, lr: float) -> Optimizer:
            h = vp()
            _w._check(_w._lib().wkz_nn_gd_init(dtype_id(dtype), lr, ctypes.byref(h)), "GD.init")
            return Optimizer(h, dtype)

    class Adam:
        """Adam.  The reference's Zig tree has no Adam to match (its adam.zig is empty); textbook rule."""

        @staticmethod
        def init(dtype: str, lr: float = 1e-3, beta1: float = 0.9, beta2: float = 0.999, eps: "float | None" = None) -> Optimizer:
            h = vp()
            _w._check(_w._lib().wkz_nn_adam_init(dtype_id(dtype), lr, beta1, beta2, -1.0 if eps is None else eps,
                                                 ctypes.byref(h)), "Adam.init")
            return Optimizer(h, dtype)


class math:
    """wekua.math.basic (src/math/basic.zig): the three functions the training step uses."""

    @staticmethod
    def dot(pipeline, x, y) -> None:
        """x = x * y element-wise, in place."""
        _w._check(_w._lib().wkz_math_dot(pipeline._h, x._h, y._h), "math.dot")

    @staticmethod
    def _reduce(fn, pipeline, x):
        out = np.zeros(1, dtype=real_np_dtype(x.dtype))
        _w._check(fn(pipeline._h, x._h, out.ctypes.data), "math.sum")
        return out[0]

    @staticmethod
    def sum(pipeline, x):
        return math._reduce(_w._lib().wkz_math_sum, pipeline, x)

    @staticmethod
    def mean(pipeline, x):
        return math._reduce(_w._lib().wkz_math_mean, pipeline, x)
