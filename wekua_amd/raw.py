"""Thin numpy helpers over the raw C ABI (device buffers, uploads, the two hot-path calls).

Used by bench.py and by the parity tests that drive `wk_gemm` / `wk_axpy` directly.
Everything here goes through libwekua_hip.so; nothing computes on the host.
"""
from __future__ import annotations

import ctypes

import numpy as np

from . import _capi
from ._capi import check

REAL_NAMES = ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64", "f32", "f64"]
DTYPE_NAMES = REAL_NAMES + ["c" + n for n in REAL_NAMES]
_NP_REAL = [np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64,
            np.float32, np.float64]


def dtype_id(name: str) -> int:
    return DTYPE_NAMES.index(name)


def real_np_dtype(name: str) -> np.dtype:
    return np.dtype(_NP_REAL[dtype_id(name) % 10])


def is_complex(name: str) -> bool:
    return name.startswith("c")


def elem_size(name: str) -> int:
    return real_np_dtype(name).itemsize * (2 if is_complex(name) else 1)


def scalar_bytes(name: str, value):
    """ctypes buffer holding one element of dtype `name`, or None for an absent scalar."""
    if value is None:
        return None
    rd = real_np_dtype(name)
    if is_complex(name):
        if isinstance(value, complex):
            value = (value.real, value.imag)
        vals = list(value)
    else:
        vals = [value]
    if rd.kind in "iu":
        mask = (1 << (8 * rd.itemsize)) - 1
        arr = np.array([int(v) & mask for v in vals], dtype=np.uint64).astype(
            np.dtype("u%d" % rd.itemsize)).view(rd)
    else:
        arr = np.array(vals, dtype=rd)
    return ctypes.create_string_buffer(arr.tobytes(), arr.nbytes)


class Device:
    """One GPU and one in-order stream on it."""

    def __init__(self, ordinal: int = 0):
        self.lib = _capi.load()
        self.dev = ctypes.c_void_p()
        check(self.lib.wk_device_open(ordinal, ctypes.byref(self.dev)), "wk_device_open")
        self.stream = ctypes.c_void_p()
        check(self.lib.wk_stream_create(self.dev, ctypes.byref(self.stream)), "wk_stream_create")
        self._live = []

    def props(self) -> _capi.WkProps:
        p = _capi.WkProps()
        check(self.lib.wk_device_props(self.dev, ctypes.byref(p)), "wk_device_props")
        return p

    def sync(self) -> None:
        check(self.lib.wk_stream_sync(self.stream), "wk_stream_sync")

    def malloc(self, nbytes: int) -> "DeviceBuffer":
        return DeviceBuffer(self, nbytes)

    def upload(self, arr: np.ndarray) -> "DeviceBuffer":
        arr = np.ascontiguousarray(arr)
        buf = DeviceBuffer(self, max(arr.nbytes, 1))
        check(self.lib.wk_copy_h2d_rect_async(self.stream, buf.ptr, arr.nbytes, 0, arr.ctypes.data, arr.nbytes, 0,
                                              arr.nbytes, 1, 1), "upload")
        self.sync()
        return buf

    def close(self) -> None:
        if self.stream:
            self.lib.wk_stream_destroy(self.stream)
            self.stream = None
        if self.dev:
            self.lib.wk_device_close(self.dev)
            self.dev = None

    def time_stream_ms(self, enqueue, iters: int) -> float:
        """Average duration in ms of `iters` calls of enqueue() measured with events recorded on
        this device's stream (the stream the kernels are launched on)."""
        e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
        check(self.lib.wk_event_create(self.dev, ctypes.byref(e0)), "wk_event_create")
        check(self.lib.wk_event_create(self.dev, ctypes.byref(e1)), "wk_event_create")
        try:
            check(self.lib.wk_event_record(e0, self.stream), "wk_event_record")
            for _ in range(iters):
                enqueue()
            check(self.lib.wk_event_record(e1, self.stream), "wk_event_record")
            check(self.lib.wk_event_sync(e1), "wk_event_sync")
            ms = ctypes.c_float()
            check(self.lib.wk_event_elapsed_ms(e0, e1, ctypes.byref(ms)), "wk_event_elapsed_ms")
        finally:
            self.lib.wk_event_destroy(e0)
            self.lib.wk_event_destroy(e1)
        return ms.value / iters

    # -- the hot path ---------------------------------------------------------------------
    def gemm(self, dtype: str, op_a: int, op_b: int, M: int, N: int, K: int, alpha, A: "DeviceBuffer", lda: int,
             B: "DeviceBuffer", ldb: int, beta, C: "DeviceBuffer", ldc: int, workspace: "DeviceBuffer | None" = None,
             b_kept: bool = False) -> None:
        """wk_gemm; b_kept: wk_gemm_packed_b_kept (the workspace still holds B's packed form)."""
        a, b = scalar_bytes(dtype, alpha), scalar_bytes(dtype, beta)
        entry = self.lib.wk_gemm_packed_b_kept if b_kept else self.lib.wk_gemm
        check(entry(self.stream, dtype_id(dtype), op_a, op_b, M, N, K,
                    ctypes.cast(a, ctypes.c_void_p) if a is not None else None, A.ptr, lda, B.ptr, ldb,
                    ctypes.cast(b, ctypes.c_void_p) if b is not None else None, C.ptr, ldc,
                    workspace.ptr if workspace is not None else None, workspace.nbytes if workspace is not None else 0),
              "wk_gemm")

    def axpy(self, dtype: str, shape3, x: "DeviceBuffer", xrp: int, xsp: int, alpha, y: "DeviceBuffer", yrp: int,
             ysp: int) -> None:
        a = scalar_bytes(dtype, alpha)
        s3 = (ctypes.c_uint64 * 3)(*shape3)
        check(self.lib.wk_axpy(self.stream, dtype_id(dtype), s3, x.ptr, xrp, xsp, y.ptr, yrp, ysp,
                               ctypes.cast(a, ctypes.c_void_p) if a is not None else None), "wk_axpy")


class DeviceBuffer:
    def __init__(self, device: Device, nbytes: int):
        self.device = device
        self.nbytes = nbytes
        self.ptr = ctypes.c_void_p()
        check(device.lib.wk_malloc(device.dev, nbytes, ctypes.byref(self.ptr)), "wk_malloc")

    def download(self, dtype: np.dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        d = self.device
        check(d.lib.wk_copy_d2h_rect_async(d.stream, out.ctypes.data, out.nbytes, 0, self.ptr, out.nbytes, 0,
                                           out.nbytes, 1, 1), "download")
        d.sync()
        return out

    def write(self, arr: np.ndarray) -> None:
        arr = np.ascontiguousarray(arr)
        d = self.device
        check(d.lib.wk_copy_h2d_rect_async(d.stream, self.ptr, arr.nbytes, 0, arr.ctypes.data, arr.nbytes, 0,
                                           arr.nbytes, 1, 1), "write")
        d.sync()

    def free(self) -> None:
        if self.ptr:
            check(self.device.lib.wk_free(self.device.dev, self.ptr), "wk_free")
            self.ptr = None

    def __del__(self):
        try:
            if self.ptr and self.device.dev:
                self.device.lib.wk_free(self.device.dev, self.ptr)
        except Exception:
            pass
