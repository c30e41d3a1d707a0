"""wekua_amd -- wekua's BLAS hot path (blas.gemm, blas.axpy) on AMD Instinct MI355X.

Layers, bottom up:

* ``libwekua_hip.so``  -- hand-written HIP kernels for gfx950 behind the C ABI of
  ``include/wekua_hip.h`` (``wekua_amd/csrc``).
* ``libwekua_host.so`` -- the host side of the reference's API (Context, Pipeline, Tensor,
  blas.gemm / blas.axpy / GemmPackedTensors, memory, fill, identity) as C++ templates
  (``wekua_amd/host/wekua.hpp``) with flat C entry points for this binding.
* this module -- a thin Python binding of those entry points that keeps the reference's names
  and argument order, so that tests read like the reference's own Zig tests:

      ctx = Context.initFromDeviceType(DeviceType.all)
      pipeline = Pipeline.init(ctx.command_queues[0])
      a = Tensor.alloc("f32", ctx, pipeline, (m, k))
      memory.readFromBuffer(pipeline, a, host_array)
      blas.gemm(pipeline, alpha, a, blas.Operation.no_transpose, b, blas.Operation.transpose, beta, c, None)
      memory.writeToBuffer(pipeline, c, out); pipeline.waitAndCleanup()

Zig errors surface as ``WekuaError`` whose ``.name`` is the Zig error name
(``InvalidValue``, ``UnqualTensorsShape``, ...).  There is no CPU fallback anywhere: a
missing native library raises at import of the symbol that needs it.
"""
from __future__ import annotations

import ctypes
import enum
import os

import numpy as np

from . import _capi
from ._capi import WkError as WekuaError  # noqa: F401  (re-export)
from .raw import DTYPE_NAMES, dtype_id, elem_size, is_complex, real_np_dtype, scalar_bytes

_PKG = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_PKG, "libwekua_host.so")

u64, vp, ci = ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int
u64p = ctypes.POINTER(u64)


class _TensorInfo(ctypes.Structure):
    _fields_ = [
        ("dtype", ci), ("ndim", ci), ("shape", u64 * 8), ("pitches", u64 * 8),
        ("number_of_elements", u64), ("number_of_elements_without_padding", u64),
        ("row_pitch", u64), ("row_pitch_for_vectors", u64), ("slice_pitch", u64),
        ("slice_pitch_for_vectors", u64), ("number_of_vectors", u64), ("size", u64),
        ("vectors_enabled", ci), ("gemm_algorithm", ci), ("buffer", vp),
    ]


HOST_SIGNATURES = {
    "wkz_context_init_from_device_type": (ci, [ci, ctypes.POINTER(vp)]),
    "wkz_context_init_from_best_device": (ci, [ci, ctypes.POINTER(vp)]),
    "wkz_context_init": (ci, [ci, ctypes.POINTER(vp)]),
    "wkz_context_deinit": (None, [vp]),
    "wkz_context_num_queues": (ci, [vp]),
    "wkz_context_stream": (vp, [vp, ci]),
    "wkz_context_device": (vp, [vp]),
    "wkz_pipeline_init": (ci, [vp, ci, ctypes.POINTER(vp)]),
    "wkz_pipeline_deinit": (None, [vp]),
    "wkz_pipeline_prealloc": (ci, [vp, u64]),
    "wkz_pipeline_wait_and_cleanup": (ci, [vp]),
    "wkz_pipeline_pending": (u64, [vp]),
    "wkz_pipeline_prev_events": (u64, [vp]),
    "wkz_pipeline_clear": (None, [vp]),
    "wkz_tensor_alloc": (ci, [vp, vp, ci, u64p, ci, ci, ctypes.POINTER(vp)]),
    "wkz_tensor_empty": (ci, [vp, vp, ci, u64p, ci, ci, ctypes.POINTER(vp)]),
    "wkz_tensor_release": (ci, [vp, vp]),
    "wkz_tensor_get_info": (ci, [vp, ctypes.POINTER(_TensorInfo)]),
    "wkz_read_from_buffer": (ci, [vp, vp, vp, u64]),
    "wkz_write_to_buffer": (ci, [vp, vp, vp, u64]),
    "wkz_fill_zeroes": (ci, [vp, vp]),
    "wkz_fill_one": (ci, [vp, vp]),
    "wkz_fill_constant": (ci, [vp, vp, vp]),
    "wkz_identity": (ci, [vp, vp]),
    "wkz_axpy": (ci, [vp, vp, vp, vp]),
    "wkz_axpy_repeat": (ci, [vp, vp, vp, vp, ctypes.c_uint32]),
    "wkz_gemm_repeat": (ci, [vp, vp, vp, ci, vp, ci, vp, vp, vp, ctypes.c_uint32]),
    "wkz_packed_init": (ci, [vp, vp, u64, ci, ctypes.POINTER(vp)]),
    "wkz_packed_init_with_dimensions": (ci, [vp, ci, u64, u64, u64, ci, ci, ctypes.POINTER(vp)]),
    "wkz_packed_deinit": (ci, [vp, vp]),
    "wkz_packed_workspace_bytes": (ci, [vp, u64p]),
    "wkz_packed_pack": (ci, [vp, vp, vp, ci, vp, ci]),
    "wkz_packed_keep_b": (ci, [vp, ci]),
    "wkz_packed_invalidate_b": (ci, [vp]),
    "wkz_gemm": (ci, [vp, vp, vp, ci, vp, ci, vp, vp, vp]),
    # tensor support operations
    "wkz_memory_copy": (ci, [vp, vp, vp]),
    "wkz_get_value": (ci, [vp, vp, u64p, u64, vp]),
    "wkz_put_value": (ci, [vp, vp, u64p, u64, vp]),
    "wkz_transpose": (ci, [vp, vp, vp, u64, u64]),
    "wkz_random_uniform": (ci, [vp, vp, u64p, vp, vp]),
    "wkz_to_complex": (ci, [vp, vp, vp, ci]),
    "wkz_to_real": (ci, [vp, vp, vp, ci]),
    "wkz_print": (ci, [vp, vp, ctypes.c_char_p, u64, u64p]),
    # math / nn (the MLP training step)
    "wkz_math_dot": (ci, [vp, vp, vp]),
    "wkz_math_sum": (ci, [vp, vp, vp]),
    "wkz_math_mean": (ci, [vp, vp, vp]),
    "wkz_nn_activation_run": (ci, [ci, vp, vp]),
    "wkz_nn_activation_get_derivative": (ci, [ci, vp, vp, vp]),
    "wkz_nn_linear_init": (ci, [vp, vp, ci, u64, u64, ci, u64, ci, u64p, ctypes.POINTER(vp)]),
    "wkz_nn_sequential_init": (ci, [ci, ctypes.POINTER(vp)]),
    "wkz_nn_sequential_append": (ci, [vp, vp]),
    "wkz_nn_layer_deinit": (ci, [vp, vp]),
    "wkz_nn_layer_tensor": (ci, [vp, vp, ci, u64, u64p, ctypes.POINTER(vp)]),
    "wkz_tensor_handle_drop": (None, [vp]),
    "wkz_nn_layer_forward": (ci, [vp, vp, vp, vp, ctypes.POINTER(vp)]),
    "wkz_nn_layer_backward": (ci, [vp, vp, vp, vp, vp]),
    "wkz_nn_cache_init": (ci, [vp, vp, u64, ctypes.POINTER(vp), u64, ctypes.POINTER(vp)]),
    "wkz_nn_cache_deinit": (ci, [vp, vp]),
    "wkz_nn_cache_get_layer_cache": (vp, [vp, u64]),
    "wkz_nn_cache_error_tensor": (ci, [vp, ctypes.POINTER(vp)]),
    "wkz_nn_loss_mse": (ci, [ci, vp, vp, vp, vp, vp]),
    "wkz_nn_gd_init": (ci, [ci, ctypes.c_double, ctypes.POINTER(vp)]),
    "wkz_nn_adam_init": (ci, [ci, ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.POINTER(vp)]),
    "wkz_nn_optimizer_step": (ci, [vp, vp, vp]),
    "wkz_nn_optimizer_zero": (ci, [vp, vp]),
    "wkz_nn_optimizer_deinit": (ci, [vp, vp]),
}

_host = None


def _lib():
    global _host
    if _host is None:
        _capi.load()  # libwekua_hip.so first (RTLD_GLOBAL): the host library links against it
        if not os.path.exists(HOST_LIB_PATH):
            raise ImportError(f"{HOST_LIB_PATH} is missing: build it with `python -m wekua_amd.build`")
        lib = ctypes.CDLL(HOST_LIB_PATH)
        for name, (res, args) in HOST_SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _host = lib
    return _host


def _check(code: int, where: str) -> None:
    if code != 0:
        raise WekuaError(code, where)


def _scalar_ptr(dtype: str, value):
    buf = scalar_bytes(dtype, value)
    return buf, (ctypes.cast(buf, vp) if buf is not None else None)


class DeviceType(enum.IntEnum):
    cpu = 0
    gpu = 1
    all = 2


class CommandQueue:
    def __init__(self, context: "Context", index: int):
        self.context = context
        self.wekua_id = index

    def isTypeSupported(self, dtype: str) -> bool:
        return dtype in DTYPE_NAMES


class Context:
    """core.Context (src/core/context.zig): one HIP device, one in-order queue."""

    def __init__(self, handle):
        self._h = handle
        n = _lib().wkz_context_num_queues(handle)
        self.command_queues = [CommandQueue(self, i) for i in range(n)]

    @classmethod
    def initFromDeviceType(cls, device_type: DeviceType = DeviceType.all) -> "Context":
        h = vp()
        _check(_lib().wkz_context_init_from_device_type(int(device_type), ctypes.byref(h)), "Context.initFromDeviceType")
        return cls(h)

    @classmethod
    def initFromBestDevice(cls, device_type: DeviceType = DeviceType.gpu) -> "Context":
        h = vp()
        _check(_lib().wkz_context_init_from_best_device(int(device_type), ctypes.byref(h)), "Context.initFromBestDevice")
        return cls(h)

    @classmethod
    def init(cls, ordinal: int = 0) -> "Context":
        h = vp()
        _check(_lib().wkz_context_init(ordinal, ctypes.byref(h)), "Context.init")
        return cls(h)

    def deinit(self) -> None:
        if self._h:
            _lib().wkz_context_deinit(self._h)
            self._h = None


class Pipeline:
    """core.Pipeline (src/core/pipeline.zig)."""

    def __init__(self, handle, command_queue: CommandQueue):
        self._h = handle
        self.command_queue = command_queue

    @classmethod
    def init(cls, command_queue: CommandQueue) -> "Pipeline":
        h = vp()
        _check(_lib().wkz_pipeline_init(command_queue.context._h, command_queue.wekua_id, ctypes.byref(h)), "Pipeline.init")
        return cls(h, command_queue)

    def deinit(self) -> None:
        if self._h:
            _lib().wkz_pipeline_deinit(self._h)
            self._h = None

    def prealloc(self, capacity: int) -> None:
        _check(_lib().wkz_pipeline_prealloc(self._h, capacity), "Pipeline.prealloc")

    def waitAndCleanup(self) -> None:
        _check(_lib().wkz_pipeline_wait_and_cleanup(self._h), "Pipeline.waitAndCleanup")
        self._keepalive = []

    def pending(self) -> int:
        return int(_lib().wkz_pipeline_pending(self._h))

    def prevEvents(self) -> int:
        """Number of events in the last appended batch (0 when nothing is pending)."""
        return int(_lib().wkz_pipeline_prev_events(self._h))

    def clear(self) -> None:
        _lib().wkz_pipeline_clear(self._h)


class Tensor:
    """Tensor(T) (src/tensor/main.zig): `dtype` plays the role of the comptime type."""

    def __init__(self, handle, dtype: str, context: Context):
        self._h = handle
        self.dtype = dtype
        self.context = context
        info = _TensorInfo()
        _check(_lib().wkz_tensor_get_info(handle, ctypes.byref(info)), "Tensor info")
        nd = info.ndim
        self.shape = tuple(int(info.shape[i]) for i in range(nd))
        self.pitches = tuple(int(info.pitches[i]) for i in range(nd))
        self.number_of_elements = int(info.number_of_elements)
        self.number_of_elements_without_padding = int(info.number_of_elements_without_padding)
        self.row_pitch = int(info.row_pitch)
        self.row_pitch_for_vectors = int(info.row_pitch_for_vectors)
        self.slice_pitch = int(info.slice_pitch)
        self.slice_pitch_for_vectors = int(info.slice_pitch_for_vectors)
        self.number_of_vectors = int(info.number_of_vectors)
        self.size = int(info.size)
        self.vectors_enabled = bool(info.vectors_enabled)
        self.gemm_algorithm = int(info.gemm_algorithm)
        self.buffer = info.buffer

    @classmethod
    def _create(cls, fn, dtype, context, pipeline, shape, vectors_enabled):
        arr = (u64 * max(len(shape), 1))(*shape)
        h = vp()
        _check(fn(context._h, pipeline._h, dtype_id(dtype), arr, len(shape), int(vectors_enabled), ctypes.byref(h)),
               "Tensor.alloc")
        return cls(h, dtype, context)

    @classmethod
    def alloc(cls, dtype: str, context: Context, pipeline: Pipeline, shape, vectors_enabled: bool = True) -> "Tensor":
        return cls._create(_lib().wkz_tensor_alloc, dtype, context, pipeline, tuple(shape), vectors_enabled)

    @classmethod
    def empty(cls, dtype: str, context: Context, pipeline: Pipeline, shape, vectors_enabled: bool = True) -> "Tensor":
        return cls._create(_lib().wkz_tensor_empty, dtype, context, pipeline, tuple(shape), vectors_enabled)

    def release(self, pipeline: Pipeline) -> None:
        if self._h:
            if getattr(self, "_borrowed", False):
                raise ValueError("this tensor belongs to a layer or cache; release that instead")
            _check(_lib().wkz_tensor_release(self._h, pipeline._h), "Tensor.release")
            self._h = None

    @classmethod
    def _borrow(cls, handle, dtype: str, context: Context) -> "Tensor":
        """View of a tensor owned by a layer or a cache; only the handle wrapper is dropped."""
        t = cls(handle, dtype, context)
        t._borrowed = True
        return t

    def __del__(self):
        if getattr(self, "_borrowed", False) and self._h and _host is not None:
            _host.wkz_tensor_handle_drop(self._h)
            self._h = None

    def host_shape(self):
        return self.shape + ((2,) if is_complex(self.dtype) else ())


class memory:
    @staticmethod
    def readFromBuffer(pipeline: Pipeline, tensor: Tensor, buffer: np.ndarray) -> None:
        """HOST -> DEVICE; `buffer` holds exactly the logical elements (complex: trailing (re, im) axis)."""
        buffer = np.ascontiguousarray(buffer, dtype=real_np_dtype(tensor.dtype))
        n = buffer.size // (2 if is_complex(tensor.dtype) else 1)
        _check(_lib().wkz_read_from_buffer(pipeline._h, tensor._h, buffer.ctypes.data, n), "memory.readFromBuffer")
        pipeline._keepalive = getattr(pipeline, "_keepalive", []) + [buffer]

    @staticmethod
    def writeToBuffer(pipeline: Pipeline, tensor: Tensor, buffer: np.ndarray) -> None:
        """DEVICE -> HOST into a C-contiguous array of the tensor's dtype."""
        if buffer.dtype != real_np_dtype(tensor.dtype) or not buffer.flags.c_contiguous:
            raise TypeError("writeToBuffer needs a C-contiguous array of the tensor's dtype")
        n = buffer.size // (2 if is_complex(tensor.dtype) else 1)
        _check(_lib().wkz_write_to_buffer(pipeline._h, tensor._h, buffer.ctypes.data, n), "memory.writeToBuffer")


    @staticmethod
    def copy(pipeline: Pipeline, src: Tensor, dst: Tensor) -> None:
        """memory.copy (src/tensor/memory/copy.zig): DEVICE -> DEVICE of the logical region."""
        _check(_lib().wkz_memory_copy(pipeline._h, src._h, dst._h), "memory.copy")

    @staticmethod
    def getValue(pipeline: Pipeline, tensor: Tensor, coor, scalar: np.ndarray) -> None:
        """memory.getValue: non-blocking read of one element into `scalar` (a 1-element array of the
        tensor's dtype; complex: 2 elements), valid after pipeline.waitAndCleanup()."""
        c = (u64 * max(len(coor), 1))(*coor)
        if scalar.dtype != real_np_dtype(tensor.dtype) or scalar.size != (2 if is_complex(tensor.dtype) else 1):
            raise TypeError("getValue needs an array holding exactly one element of the tensor's dtype")
        _check(_lib().wkz_get_value(pipeline._h, tensor._h, c, len(coor), scalar.ctypes.data), "memory.getValue")

    @staticmethod
    def putValue(pipeline: Pipeline, tensor: Tensor, coor, value) -> None:
        """memory.putValue: write one element."""
        c = (u64 * max(len(coor), 1))(*coor)
        keep, p = _scalar_ptr(tensor.dtype, value)
        _check(_lib().wkz_put_value(pipeline._h, tensor._h, c, len(coor), p), "memory.putValue")
        pipeline._keepalive = getattr(pipeline, "_keepalive", []) + [keep]


class fill:
    @staticmethod
    def zeroes(pipeline: Pipeline, tensor: Tensor) -> None:
        _check(_lib().wkz_fill_zeroes(pipeline._h, tensor._h), "fill.zeroes")

    @staticmethod
    def one(pipeline: Pipeline, tensor: Tensor) -> None:
        _check(_lib().wkz_fill_one(pipeline._h, tensor._h), "fill.one")

    @staticmethod
    def constant(pipeline: Pipeline, tensor: Tensor, value) -> None:
        _keep, p = _scalar_ptr(tensor.dtype, value)
        _check(_lib().wkz_fill_constant(pipeline._h, tensor._h, p), "fill.constant")


def identity(pipeline: Pipeline, tensor: Tensor) -> None:
    _check(_lib().wkz_identity(pipeline._h, tensor._h), "identity")


def transpose(pipeline: Pipeline, result_tensor: Tensor, tensor: Tensor, dim0: int, dim1: int) -> None:
    """tensor.transpose (src/tensor/transpose.zig): result = tensor with dim0 and dim1 exchanged."""
    _check(_lib().wkz_transpose(pipeline._h, result_tensor._h, tensor._h, dim0, dim1), "transpose")


def printZ(pipeline: Pipeline, tensor: Tensor) -> str:
    """tensor.printZ (src/tensor/print.zig): the text `print` writes."""
    need = u64()
    _check(_lib().wkz_print(pipeline._h, tensor._h, None, 0, ctypes.byref(need)), "printZ")
    buf = ctypes.create_string_buffer(need.value + 1)
    _check(_lib().wkz_print(pipeline._h, tensor._h, buf, need.value + 1, None), "printZ")
    return buf.value.decode()


def print_tensor(pipeline: Pipeline, tensor: Tensor) -> None:
    """tensor.print (`print` is taken in Python)."""
    import sys
    sys.stdout.write(printZ(pipeline, tensor))


class Space(enum.IntEnum):
    real = 0
    imag = 1


class random:
    @staticmethod
    def uniform(pipeline: Pipeline, tensor: Tensor, seed=None, min_value=None, max_value=None) -> None:
        """random.uniform (src/tensor/random/uniform.zig): seed None draws it from the clock; without
        min/max floats land in [0, 1] and integers take the low bits of the hash."""
        sub = DTYPE_NAMES[dtype_id(tensor.dtype) % 10]
        seed_arg = ctypes.byref(u64(seed)) if seed is not None else None
        _k1, pmin = _scalar_ptr(sub, min_value)
        _k2, pmax = _scalar_ptr(sub, max_value)
        _check(_lib().wkz_random_uniform(pipeline._h, tensor._h, seed_arg, pmin, pmax), "random.uniform")

    @staticmethod
    def hash(index: int, seed: int) -> int:
        """The 64-bit hash random.uniform draws from."""
        return int(_capi.load().wk_random_hash(index, seed))


class convertions:
    @staticmethod
    def toComplex(pipeline: Pipeline, src: Tensor, dst: Tensor, space: Space) -> None:
        _check(_lib().wkz_to_complex(pipeline._h, src._h, dst._h, int(space)), "toComplex")

    @staticmethod
    def toReal(pipeline: Pipeline, src: Tensor, dst: Tensor, space: Space) -> None:
        _check(_lib().wkz_to_real(pipeline._h, src._h, dst._h, int(space)), "toReal")


class GemmPackedTensors:
    """blas.GemmPackedTensors (src/blas/gemm.zig:60-359).  Holds device memory only for the types
    whose gemm has a pack pass (8/16/32-bit integers, their complex types, cf32, cf64): its workspace
    (`workspace_bytes`).
    keepB / invalidateB have no counterpart in the reference, which packs both operands on every
    call: they let a constant B (weights) stay packed across calls."""

    def __init__(self, handle, dtype):
        self._h = handle
        self.dtype = dtype

    @property
    def workspace_bytes(self) -> int:
        n = u64()
        _check(_lib().wkz_packed_workspace_bytes(self._h, ctypes.byref(n)), "GemmPackedTensors.workspace_bytes")
        return n.value

    @classmethod
    def init(cls, pipeline: Pipeline, result_tensor: Tensor, k_size: int, vectors_enabled: bool) -> "GemmPackedTensors":
        h = vp()
        _check(_lib().wkz_packed_init(pipeline._h, result_tensor._h, k_size, int(vectors_enabled), ctypes.byref(h)),
               "GemmPackedTensors.init")
        return cls(h, result_tensor.dtype)

    @classmethod
    def initWithDimensions(cls, pipeline: Pipeline, dtype: str, n_size: int, m_size: int, k_size: int,
                           recommended_algorithm: int, vectors_enabled: bool) -> "GemmPackedTensors":
        h = vp()
        _check(_lib().wkz_packed_init_with_dimensions(pipeline._h, dtype_id(dtype), n_size, m_size, k_size,
                                                      recommended_algorithm, int(vectors_enabled), ctypes.byref(h)),
               "GemmPackedTensors.initWithDimensions")
        return cls(h, dtype)

    def deinit(self, pipeline: Pipeline) -> None:
        if self._h:
            _check(_lib().wkz_packed_deinit(self._h, pipeline._h), "GemmPackedTensors.deinit")
            self._h = None

    def keepB(self, on: bool) -> None:
        """While on, gemm calls after the first with the same B tensor, op_b, pipeline queue and alpha
        skip B's pack pass; call invalidateB() after B's contents change."""
        _check(_lib().wkz_packed_keep_b(self._h, int(on)), "GemmPackedTensors.keepB")

    def invalidateB(self) -> None:
        _check(_lib().wkz_packed_invalidate_b(self._h), "GemmPackedTensors.invalidateB")

    def pack(self, pipeline: Pipeline, a: Tensor, op_a: int, b: Tensor, op_b: int) -> None:
        _check(_lib().wkz_packed_pack(self._h, pipeline._h, a._h, int(op_a), b._h, int(op_b)), "GemmPackedTensors.pack")


class blas:
    class Operation(enum.IntEnum):
        no_transpose = 0
        transpose = 1

    GemmOperation = Operation
    GemmPackedTensors = GemmPackedTensors

    @staticmethod
    def axpy(pipeline: Pipeline, x: Tensor, alpha, y: Tensor) -> None:
        """blas.axpy(T, pipeline, x, alpha, y): y = alpha*x + y (alpha None: y += x)."""
        _keep, p = _scalar_ptr(x.dtype, alpha)
        _check(_lib().wkz_axpy(pipeline._h, x._h, p, y._h), "blas.axpy")

    @staticmethod
    def axpy_repeat(pipeline: Pipeline, x: Tensor, alpha, y: Tensor, count: int) -> None:
        """blas.axpy `count` times from one loop inside the host library (benchmarks: a call from Python costs more
        interpreter time than a short launch takes)."""
        _keep, p = _scalar_ptr(x.dtype, alpha)
        _check(_lib().wkz_axpy_repeat(pipeline._h, x._h, p, y._h, int(count)), "blas.axpy")

    @staticmethod
    def gemm_repeat(pipeline: Pipeline, alpha, a: Tensor, op_a: int, b: Tensor, op_b: int, beta, c: Tensor,
                    packed_tensors: "GemmPackedTensors | None", count: int) -> None:
        """blas.gemm `count` times from one loop inside the host library (benchmarks)."""
        _ka, pa = _scalar_ptr(c.dtype, alpha)
        _kb, pb = _scalar_ptr(c.dtype, beta)
        _check(_lib().wkz_gemm_repeat(pipeline._h, pa, a._h, int(op_a), b._h, int(op_b), pb, c._h,
                                      packed_tensors._h if packed_tensors is not None else None, int(count)), "blas.gemm")

    @staticmethod
    def gemm(pipeline: Pipeline, alpha, a: Tensor, op_a: int, b: Tensor, op_b: int, beta, c: Tensor,
             packed_tensors: "GemmPackedTensors | None" = None) -> None:
        """blas.gemm(T, pipeline, alpha, a, op_a, b, op_b, beta, c, packed_tensors)."""
        _ka, pa = _scalar_ptr(c.dtype, alpha)
        _kb, pb = _scalar_ptr(c.dtype, beta)
        _check(_lib().wkz_gemm(pipeline._h, pa, a._h, int(op_a), b._h, int(op_b), pb, c._h,
                               packed_tensors._h if packed_tensors is not None else None), "blas.gemm")


from . import nn  # noqa: E402  (needs the classes above)
from .nn import math  # noqa: E402,F401

__all__ = ["nn", "math", "printZ", "print_tensor", "transpose", "random", "convertions", "Space", "Context", "Pipeline", "Tensor", "CommandQueue", "DeviceType", "memory", "fill", "identity", "blas",
           "GemmPackedTensors", "WekuaError", "DTYPE_NAMES", "dtype_id", "elem_size", "is_complex", "real_np_dtype"]
