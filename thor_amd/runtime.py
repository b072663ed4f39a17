"""Thin Python handles over the device-side C ABI (include/thorhip.h): streams, events, raw device buffers, and the
TypeConverter entry point.  No arithmetic happens here."""
from __future__ import annotations

import ctypes

import numpy as np

from . import _lib
from .dtypes import DataType, numpy_carrier, size_of

H2D, D2H, D2D = 1, 2, 3


def device_count() -> int:
    n = ctypes.c_int(0)
    _lib.check(_lib.load().thorhip_device_count(ctypes.byref(n)), "thorhip_device_count")
    return n.value


def set_device(device: int) -> None:
    _lib.check(_lib.load().thorhip_set_device(device), "thorhip_set_device")


def device_info(device: int = 0) -> _lib.DeviceInfo:
    info = _lib.DeviceInfo()
    _lib.check(_lib.load().thorhip_device_get_info(device, ctypes.byref(info)), "thorhip_device_get_info")
    return info


def device_synchronize() -> None:
    _lib.check(_lib.load().thorhip_device_synchronize(), "thorhip_device_synchronize")


class Stream:
    """Mirror of the reference's Stream handle (Utilities/Common/Stream.h:35-116): a HIP stream on one GPU."""

    def __init__(self, gpu_num: int = 0):
        self.gpu_num = gpu_num
        set_device(gpu_num)
        h = ctypes.c_void_p()
        _lib.check(_lib.load().thorhip_stream_create(ctypes.byref(h)), "thorhip_stream_create")
        self.handle = h

    def synchronize(self) -> None:
        _lib.check(_lib.load().thorhip_stream_synchronize(self.handle), "thorhip_stream_synchronize")

    def wait_event(self, event: "Event") -> None:
        _lib.check(_lib.load().thorhip_stream_wait_event(self.handle, event.handle), "thorhip_stream_wait_event")

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                _lib.load().thorhip_stream_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class Event:
    def __init__(self, enable_timing: bool = True):
        h = ctypes.c_void_p()
        _lib.check(_lib.load().thorhip_event_create(ctypes.byref(h), 1 if enable_timing else 0), "thorhip_event_create")
        self.handle = h

    def record(self, stream: Stream | None = None) -> None:
        _lib.check(_lib.load().thorhip_event_record(self.handle, stream.handle if stream else None), "thorhip_event_record")

    def synchronize(self) -> None:
        _lib.check(_lib.load().thorhip_event_synchronize(self.handle), "thorhip_event_synchronize")

    def elapsed_ms(self, later: "Event") -> float:
        ms = ctypes.c_float(0)
        _lib.check(_lib.load().thorhip_event_elapsed_ms(ctypes.byref(ms), self.handle, later.handle), "thorhip_event_elapsed_ms")
        return ms.value

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                _lib.load().thorhip_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class DeviceBuffer:
    """A raw device allocation of `nbytes` bytes."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        p = ctypes.c_void_p()
        _lib.check(_lib.load().thorhip_malloc(ctypes.byref(p), self.nbytes), "thorhip_malloc")
        self.ptr = p.value or 0

    @classmethod
    def from_numpy(cls, arr: np.ndarray, stream: Stream | None = None) -> "DeviceBuffer":
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.upload(arr, stream)
        return buf

    def upload(self, arr: np.ndarray, stream: Stream | None = None, offset_bytes: int = 0) -> None:
        arr = np.ascontiguousarray(arr)
        assert offset_bytes + arr.nbytes <= self.nbytes
        L = _lib.load()
        _lib.check(L.thorhip_memcpy_async(self.ptr + offset_bytes, arr.ctypes.data, arr.nbytes, H2D, stream.handle if stream else None),
                   "thorhip_memcpy_async(H2D)")
        # pageable host memory: make the copy synchronous so the numpy array may be released
        _lib.check(L.thorhip_stream_synchronize(stream.handle if stream else None), "thorhip_stream_synchronize")

    def download(self, dtype, count: int, stream: Stream | None = None, offset_bytes: int = 0) -> np.ndarray:
        out = np.empty(count, dtype=dtype)
        assert offset_bytes + out.nbytes <= self.nbytes
        L = _lib.load()
        _lib.check(L.thorhip_memcpy_async(out.ctypes.data, self.ptr + offset_bytes, out.nbytes, D2H, stream.handle if stream else None),
                   "thorhip_memcpy_async(D2H)")
        _lib.check(L.thorhip_stream_synchronize(stream.handle if stream else None), "thorhip_stream_synchronize")
        return out

    def memset(self, byte_value: int, stream: Stream | None = None) -> None:
        _lib.check(_lib.load().thorhip_memset_async(self.ptr, byte_value, self.nbytes, stream.handle if stream else None),
                   "thorhip_memset_async")

    def free(self) -> None:
        if getattr(self, "ptr", 0):
            _lib.load().thorhip_free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class TypeConverter:
    """Mirror of TypeConverter::convertType (Utilities/TensorOperations/DataTypeConversions/TypeConverter.h:30-36) for
    device memory: schedules `dest[i] = static_cast<dest dtype>(source[i])` at the back of `stream`."""

    @staticmethod
    def convert_type(source_ptr: int, dest_ptr: int, source_dtype: DataType, dest_dtype: DataType, num_elements: int,
                     stream: Stream | None = None) -> None:
        if DataType(source_dtype) == DataType(dest_dtype):
            raise ValueError("convert_type requires different source and destination dtypes")
        if num_elements < 0:
            raise ValueError("num_elements must be non-negative")
        _lib.check(_lib.load().thorhip_convert(source_ptr, dest_ptr, int(source_dtype), int(dest_dtype), int(num_elements),
                                               stream.handle if stream else None), "thorhip_convert")


def convert_array(values: np.ndarray, source_dtype: DataType, dest_dtype: DataType, stream: Stream | None = None) -> np.ndarray:
    """Round trip helper: upload a carrier array, convert on the GPU, download the carrier of the destination dtype."""
    values = np.ascontiguousarray(values)
    assert values.dtype == numpy_carrier(source_dtype), (values.dtype, source_dtype)
    n = values.size
    src = DeviceBuffer.from_numpy(values, stream)
    dst = DeviceBuffer(max(1, n * size_of(dest_dtype)))
    TypeConverter.convert_type(src.ptr, dst.ptr, source_dtype, dest_dtype, n, stream)
    out = dst.download(numpy_carrier(dest_dtype), n, stream).reshape(values.shape)
    src.free()
    dst.free()
    return out
