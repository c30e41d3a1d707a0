"""ctypes binding of the C ABI declared in include/wekua_hip.h (libwekua_hip.so).

The library is loaded from the package directory (built in-tree by wekua_amd/build.py).
There is no CPU fallback: if the library is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libwekua_hip.so")

u64 = ctypes.c_uint64
vp = ctypes.c_void_p
ci = ctypes.c_int
sz = ctypes.c_size_t
u64p = ctypes.POINTER(u64)


class WkProps(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 64),
        ("arch", ctypes.c_char * 32),
        ("ordinal", ci),
        ("compute_units", ci),
        ("wavefront_size", ci),
        ("max_work_group_size", ci),
        ("local_mem_bytes", u64),
        ("global_mem_bytes", u64),
        ("cache_line_size", ci),
        ("clock_mhz", ci),
    ]


class WkAdamTensor(ctypes.Structure):
    """wk_adam_tensor of include/wekua_hip.h"""
    _fields_ = [("w", ctypes.c_void_p), ("g", ctypes.c_void_p), ("m", ctypes.c_void_p), ("v", ctypes.c_void_p),
                ("shape3", ctypes.c_uint64 * 3), ("w_row_pitch", ctypes.c_uint64), ("w_slice_pitch", ctypes.c_uint64),
                ("g_row_pitch", ctypes.c_uint64), ("g_slice_pitch", ctypes.c_uint64), ("mv_row_pitch", ctypes.c_uint64),
                ("mv_slice_pitch", ctypes.c_uint64)]


# name -> (restype, argtypes); one entry per declaration in include/wekua_hip.h and include/wekua_hip_test.h
SIGNATURES = {
    "wk_strerror": (ctypes.c_char_p, [ci]),
    "wk_abi_version": (ci, []),
    "wk_dtype_size": (sz, [ci]),
    "wk_device_count": (ci, [ctypes.POINTER(ci)]),
    "wk_device_open": (ci, [ci, ctypes.POINTER(vp)]),
    "wk_device_close": (None, [vp]),
    "wk_device_props": (ci, [vp, ctypes.POINTER(WkProps)]),
    "wk_stream_create": (ci, [vp, ctypes.POINTER(vp)]),
    "wk_stream_destroy": (None, [vp]),
    "wk_stream_sync": (ci, [vp]),
    "wk_stream_native": (vp, [vp]),
    "wk_event_create": (ci, [vp, ctypes.POINTER(vp)]),
    "wk_event_destroy": (None, [vp]),
    "wk_event_record": (ci, [vp, vp]),
    "wk_event_sync": (ci, [vp]),
    "wk_event_elapsed_ms": (ci, [vp, vp, ctypes.POINTER(ctypes.c_float)]),
    "wk_malloc": (ci, [vp, sz, ctypes.POINTER(vp)]),
    "wk_free": (ci, [vp, vp]),
    "wk_mem_info": (ci, [vp, ctypes.POINTER(sz), ctypes.POINTER(sz)]),
    "wk_memset_async": (ci, [vp, vp, ci, sz]),
    "wk_copy_h2d_rect_async": (ci, [vp, vp, sz, sz, vp, sz, sz, sz, sz, sz]),
    "wk_copy_d2h_rect_async": (ci, [vp, vp, sz, sz, vp, sz, sz, sz, sz, sz]),
    "wk_copy_d2d_rect_async": (ci, [vp, vp, sz, sz, vp, sz, sz, sz, sz, sz]),
    "wk_fill": (ci, [vp, ci, vp, u64p, u64, u64, vp]),
    "wk_identity": (ci, [vp, ci, vp, u64, u64]),
    "wk_axpy": (ci, [vp, ci, u64p, vp, u64, u64, vp, u64, u64, vp]),
    "wk_gemm": (ci, [vp, ci, ci, ci, u64, u64, u64, vp, vp, u64, vp, u64, vp, vp, u64, vp, sz]),
    "wk_gemm_packed_b_kept": (ci, [vp, ci, ci, ci, u64, u64, u64, vp, vp, u64, vp, u64, vp, vp, u64, vp, sz]),
    "wk_gemm_workspace_bytes": (sz, [ci, ci, ci, u64, u64, u64]),
    "wk_gemm_variant": (ctypes.c_char_p, [ci, ci, ci, u64, u64, u64, u64, u64, u64, vp, vp, vp]),
    "wk_gemm_variant_with_workspace": (ctypes.c_char_p, [ci, ci, ci, u64, u64, u64, u64, u64, u64, vp, vp, vp, sz]),
    "wk_gemm_force_variant": (ci, [ctypes.c_char_p]),
    "wk_gemm_split_plan": (ci, [ci, ci, ci, u64, u64, u64, ctypes.c_char_p, ctypes.POINTER(ctypes.c_uint32),
                                ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(u64), ctypes.POINTER(u64),
                                ctypes.POINTER(ctypes.c_size_t)]),
    "wk_copy_kernel": (ci, [vp, vp, vp, sz]),
    "wk_stream_probe": (ci, [vp, ctypes.c_int, vp, vp, sz, ctypes.c_uint]),
    "wk_test_option": (ci, [ctypes.c_char_p, ci]),
    "wk_probe_launch": (ci, [vp, ci, ctypes.c_uint, ctypes.c_uint, sz, vp, sz]),
    "wk_hadamard": (ci, [vp, ci, u64p, vp, u64, u64, vp, u64, u64]),
    "wk_activation": (ci, [vp, ci, ci, u64p, vp, u64, u64]),
    "wk_activation_dev": (ci, [vp, ci, ci, u64p, vp, u64, u64, vp, u64, u64]),
    "wk_bias_activation": (ci, [vp, ci, ci, u64, u64, vp, u64, vp]),
    "wk_gemm_bias_activation": (ci, [vp, ci, ci, ci, u64, u64, u64, vp, u64, vp, u64, vp, u64, vp, ci]),
    "wk_bias_step": (ci, [vp, ci, u64, u64, vp, u64, vp]),
    "wk_bias_step_static": (ci, [vp, ci, u64, u64, vp, u64, vp]),
    "wk_sensitivity_step": (ci, [vp, ci, ci, u64, u64, vp, u64, vp, u64, vp, u64, vp]),
    "wk_adam_step_multi": (ci, [vp, ci, ctypes.c_uint32, vp, ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.c_double, u64]),
    "wk_mse": (ci, [vp, ci, u64p, vp, u64, u64, vp, u64, u64, vp, u64, u64, vp, u64, u64]),
    "wk_sum_workspace_bytes": (sz, [ci]),
    "wk_sum": (ci, [vp, ci, u64p, vp, u64, u64, vp, vp, ctypes.c_double]),
    "wk_adam_step": (ci, [vp, ci, u64p, vp, u64, u64, vp, u64, u64, vp, vp, u64, u64, ctypes.c_double, ctypes.c_double,
                          ctypes.c_double, ctypes.c_double, u64]),
    "wk_transpose": (ci, [vp, ci, ci, u64p, u64p, u64p, ci, ci, vp, vp]),
    "wk_random_uniform": (ci, [vp, ci, u64p, vp, u64, u64, u64, vp, vp]),
    "wk_random_hash": (u64, [u64, u64]),
    "wk_to_complex": (ci, [vp, ci, u64p, vp, u64, u64, vp, u64, u64, ci]),
    "wk_to_real": (ci, [vp, ci, u64p, vp, u64, u64, vp, u64, u64, ci]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Loads libwekua_hip.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m wekua_amd.build` "
                "(there is no CPU fallback for the GPU path)")
        lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class WkError(RuntimeError):
    def __init__(self, code: int, where: str = ""):
        self.code = code
        msg = load().wk_strerror(code).decode()
        super().__init__(f"{where}: {msg} ({code})" if where else f"{msg} ({code})")
        self.name = msg


def check(code: int, where: str = "") -> None:
    if code != 0:
        raise WkError(code, where)
