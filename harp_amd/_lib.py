"""ctypes view of libeclat_hip.so (the C ABI of include/eclat_hip.h).

The library is the only execution path: if it has not been built, importing
this module raises -- there is no CPU stand-in.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, byref, c_char, c_char_p, c_double, c_float, c_int,
                    c_size_t, c_uint, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libeclat_hip.so")

# Generated kernels are cached as gfx950 code objects next to the library unless the
# user points HARP_CACHE_DIR elsewhere (same variable as the reference's disk cache).
os.environ.setdefault("HARP_CACHE_DIR", os.path.join(_HERE, "kernel_cache"))


class EhError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `python -m harp_amd.build` "
        f"(or `__graft_entry__.build()`); the HIP backend has no fallback path")

lib = ctypes.CDLL(LIB_PATH)


class DeviceProps(Structure):
    _fields_ = [("name", c_char * 128), ("arch", c_char * 32), ("compute_units", c_int),
                ("warp_size", c_int), ("max_work_group_size", c_int),
                ("local_memory_size", c_size_t), ("global_memory_size", c_size_t),
                ("clock_khz", c_int), ("memory_clock_khz", c_int), ("memory_bus_bits", c_int),
                ("l2_bytes", c_int)]


class LaunchInfo(Structure):
    _fields_ = [("entry", c_char_p), ("source", c_char_p), ("schedule", c_char_p),
                ("grid", c_uint * 3), ("block", c_uint * 3), ("lds_bytes", c_uint),
                ("n_args", c_int), ("n_kernels", c_int), ("algo_bytes", c_double),
                ("flops", c_double), ("lane", c_int), ("n_waits", c_int), ("tune_key", ctypes.c_ulonglong)]


_P = c_void_p
_SIGS = {
    "eh_version": ([], c_int),
    "eh_last_error": ([], c_char_p),
    "eh_free": ([_P], None),
    "eh_device_count": ([POINTER(c_int)], c_int),
    "eh_device_open": ([c_int, POINTER(_P)], c_int),
    "eh_device_close": ([_P], c_int),
    "eh_device_get_props": ([_P, POINTER(DeviceProps)], c_int),
    "eh_device_sync": ([_P], c_int),
    "eh_device_stream": ([_P, POINTER(c_void_p)], c_int),
    "eh_device_trim": ([_P, POINTER(c_size_t)], c_int),
    "eh_buffer_alloc": ([_P, c_size_t, POINTER(_P)], c_int),
    "eh_buffer_retain": ([_P], c_int),
    "eh_buffer_release": ([_P], c_int),
    "eh_buffer_bytes": ([_P, POINTER(c_size_t)], c_int),
    "eh_buffer_write": ([_P, _P, c_size_t], c_int),
    "eh_buffer_read": ([_P, _P, c_size_t], c_int),
    "eh_buffer_copy": ([_P, _P], c_int),
    "eh_buffer_device_ptr": ([_P, POINTER(_P)], c_int),
    "eh_render_program": ([c_char_p, c_char_p, POINTER(_P)], c_int),
    "eh_normalize_ast": ([c_char_p, POINTER(c_void_p)], c_int),
    "eh_fit_local_size": ([POINTER(c_size_t), POINTER(c_size_t), c_size_t, POINTER(c_size_t)], c_int),
    "eh_plan_num_launches": ([_P, POINTER(c_int)], c_int),
    "eh_plan_launch": ([_P, c_int, POINTER(LaunchInfo)], c_int),
    "eh_plan_launch_arg": ([_P, c_int, c_int, POINTER(c_char_p)], c_int),
    "eh_plan_launch_kernel": ([_P, c_int, c_int, POINTER(c_char_p)], c_int),
    "eh_tune_key": ([c_char_p, POINTER(ctypes.c_ulonglong)], c_int),
    "eh_plan_launch_arg_written": ([_P, c_int, c_int, POINTER(c_int)], c_int),
    "eh_plan_launch_wait": ([_P, c_int, c_int, POINTER(c_int)], c_int),
    "eh_plan_num_buffers": ([_P, POINTER(c_int)], c_int),
    "eh_plan_buffer": ([_P, c_int, POINTER(c_char_p), POINTER(c_char_p), POINTER(c_size_t),
                        POINTER(c_int)], c_int),
    "eh_plan_release": ([_P], c_int),
    "eh_compile_source": ([c_char_p, c_char_p, POINTER(_P), POINTER(c_size_t)], c_int),
    "eh_program_compile": ([_P, c_char_p, c_char_p, POINTER(_P)], c_int),
    "eh_program_release": ([_P], c_int),
    "eh_program_num_buffers": ([_P, POINTER(c_int)], c_int),
    "eh_program_buffer": ([_P, c_int, POINTER(c_char_p), POINTER(c_char_p), POINTER(c_size_t),
                           POINTER(c_int)], c_int),
    "eh_program_num_launches": ([_P, POINTER(c_int)], c_int),
    "eh_program_launch": ([_P, c_int, POINTER(LaunchInfo)], c_int),
    "eh_program_execute": ([_P, POINTER(_P), c_int, c_int], c_int),
    "eh_program_execute_static": ([_P, POINTER(_P), c_int, c_int], c_int),
    "eh_program_record": ([_P, POINTER(_P), c_int, POINTER(_P)], c_int),
    "eh_graph_replay": ([_P, c_int], c_int),
    "eh_graph_release": ([_P], c_int),
    "eh_program_execute_positional": ([_P, POINTER(_P), c_int, POINTER(_P), c_int, c_int], c_int),
    "eh_program_binary": ([_P, c_int, POINTER(_P), POINTER(c_size_t)], c_int),
    "eh_module_load": ([_P, _P, c_size_t, c_char_p, POINTER(_P)], c_int),
    "eh_module_launch": ([_P, POINTER(c_uint), POINTER(c_uint), c_uint, POINTER(_P), c_int, c_int], c_int),
    "eh_module_release": ([_P], c_int),
    "eh_event_create": ([_P, POINTER(_P)], c_int),
    "eh_event_record": ([_P], c_int),
    "eh_event_sync": ([_P], c_int),
    "eh_event_elapsed_ms": ([_P, _P, POINTER(c_float)], c_int),
    "eh_event_release": ([_P], c_int),
}

EXPORTED = sorted(_SIGS)

for _name, (_args, _res) in _SIGS.items():
    _fn = getattr(lib, _name)      # AttributeError here = the library lacks a declared symbol
    _fn.argtypes = _args
    _fn.restype = _res


def check(code: int) -> None:
    if code != 0:
        raise EhError(code, (lib.eh_last_error() or b"").decode("utf-8", "replace"))
