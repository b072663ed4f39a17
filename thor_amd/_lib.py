"""Loads libthor_amd.so and declares the C ABI (include/thorhip.h, include/thor_c_api.h) for ctypes.

There is no fallback: if the library is missing or a symbol is absent the import fails loudly.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libthor_amd.so")


class ThorHipError(RuntimeError):
    """A thorhip_* / thor_* entry point returned a failure code."""


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("compute_units", ctypes.c_int),
        ("wavefront_size", ctypes.c_int),
        ("max_threads_per_block", ctypes.c_int),
        ("lds_bytes_per_block", ctypes.c_int),
        ("l2_bytes", ctypes.c_int),
        ("clock_khz", ctypes.c_int),
        ("memory_clock_khz", ctypes.c_int),
        ("memory_bus_width_bits", ctypes.c_int),
        ("total_global_mem", ctypes.c_size_t),
        ("arch_name", ctypes.c_char * 64),
        ("name", ctypes.c_char * 128),
    ]


_vp, _i, _i64, _sz, _u32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t, ctypes.c_uint32
_vpp = ctypes.POINTER(ctypes.c_void_p)
_ip = ctypes.POINTER(ctypes.c_int)
_szp = ctypes.POINTER(ctypes.c_size_t)
HOST_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p)

# name -> (restype, argtypes); every symbol include/thorhip.h declares
THORHIP_PROTOTYPES = {
    "thorhip_abi_version": (_i, []),
    "thorhip_last_error": (ctypes.c_char_p, []),
    "thorhip_device_count": (_i, [_ip]),
    "thorhip_set_device": (_i, [_i]),
    "thorhip_get_device": (_i, [_ip]),
    "thorhip_device_get_info": (_i, [_i, ctypes.POINTER(DeviceInfo)]),
    "thorhip_device_synchronize": (_i, []),
    "thorhip_malloc": (_i, [_vpp, _sz]),
    "thorhip_free": (_i, [_vp]),
    "thorhip_host_malloc": (_i, [_vpp, _sz]),
    "thorhip_host_free": (_i, [_vp]),
    "thorhip_memcpy_async": (_i, [_vp, _vp, _sz, _i, _vp]),
    "thorhip_memset_async": (_i, [_vp, _i, _sz, _vp]),
    "thorhip_mem_get_info": (_i, [_szp, _szp]),
    "thorhip_stream_create": (_i, [_vpp]),
    "thorhip_stream_destroy": (_i, [_vp]),
    "thorhip_stream_synchronize": (_i, [_vp]),
    "thorhip_stream_wait_event": (_i, [_vp, _vp]),
    "thorhip_stream_enqueue_host_function": (_i, [_vp, HOST_FN, _vp]),
    "thorhip_event_create": (_i, [_vpp, _i]),
    "thorhip_event_destroy": (_i, [_vp]),
    "thorhip_event_record": (_i, [_vp, _vp]),
    "thorhip_event_synchronize": (_i, [_vp]),
    "thorhip_event_elapsed_ms": (_i, [ctypes.POINTER(ctypes.c_float), _vp, _vp]),
    "thorhip_set_compile_isolation": (_i, [_i]),
    "thorhip_compile": (_i, [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_char_p), _i, _vpp, _szp,
                             ctypes.c_char_p, _sz]),
    "thorhip_code_free": (_i, [_vp]),
    "thorhip_module_load": (_i, [_vpp, _vp, _sz]),
    "thorhip_module_unload": (_i, [_vp]),
    "thorhip_module_get_function": (_i, [_vpp, _vp, ctypes.c_char_p]),
    "thorhip_function_get_attributes": (_i, [_vp, _ip, _ip, _ip]),
    "thorhip_launch": (_i, [_vp, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _vp, _vpp]),
    "thorhip_convert": (_i, [_vp, _vp, _i, _i, _i64, _vp]),
    "thorhip_dtype_size": (_i, [_i]),
}

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C thor_amd/csrc`). thor_amd has no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    for name, (restype, argtypes) in THORHIP_PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is absent
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc: int, what: str = "") -> None:
    if rc != 0:
        msg = load().thorhip_last_error()
        raise ThorHipError(f"{what} failed (code {rc}): {msg.decode('utf-8', 'replace') if msg else ''}")
