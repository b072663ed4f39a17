"""ctypes front-end of the CPU oracle (test infrastructure only).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the product
(thor_amd) never does.  The arithmetic lives in thor_oracle.c; expression evaluation lives in expr.py.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libthor_oracle.so")

FP16, FP32, FP64 = 10, 11, 12
INT8, INT16, INT32, INT64 = 13, 14, 15, 16
UINT8, UINT16, UINT32, UINT64 = 17, 18, 19, 20
BOOLEAN, FP8_E4M3, FP8_E5M2, BF16 = 21, 22, 23, 24

SUM, MIN, MAX, PRODUCT, MEAN, L1NORM, L2NORM = range(7)
ARGMIN, ARGMAX = 0, 1

# numpy carrier for every storage dtype; 16-bit brain floats and fp8 travel as raw unsigned integers
CARRIER = {
    FP16: np.float16, FP32: np.float32, FP64: np.float64,
    INT8: np.int8, INT16: np.int16, INT32: np.int32, INT64: np.int64,
    UINT8: np.uint8, UINT16: np.uint16, UINT32: np.uint32, UINT64: np.uint64,
    BOOLEAN: np.uint8, FP8_E4M3: np.uint8, FP8_E5M2: np.uint8, BF16: np.uint16,
}


def build(force: bool = False) -> str:
    """Compile libthor_oracle.so with gcc when missing (or when force is set)."""
    sources = [os.path.join(_HERE, name) for name in ("thor_oracle.c", "thor_oracle_expr.c", "thor_oracle.h")]
    stale = (not os.path.exists(_LIB_PATH)) or any(os.path.getmtime(_LIB_PATH) < os.path.getmtime(src) for src in sources)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_convert.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_long, ctypes.c_int]
        L.oracle_convert.restype = ctypes.c_int
        for name in ("oracle_check_f16_against_f16c", "oracle_check_bf16_against_addtrick", "oracle_check_f16_widen_against_f16c"):
            getattr(L, name).restype = ctypes.c_long
        u64p, u32p = ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint32)
        L.oracle_reduce.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, u64p, u64p, ctypes.c_int, u32p, ctypes.c_int,
                                    ctypes.c_float, ctypes.c_void_p, ctypes.c_int]
        L.oracle_reduce_f64.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, u64p, u64p, ctypes.c_int, u32p, ctypes.c_int,
                                        ctypes.c_void_p]
        L.oracle_arg_reduce.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, u64p, u64p, ctypes.c_int, u32p, ctypes.c_int,
                                        ctypes.c_void_p, ctypes.c_void_p]
        L.oracle_dtype_size.argtypes = [ctypes.c_int]
        vp, lg = ctypes.c_void_p, ctypes.c_long
        L.oracle_expr_config1.argtypes = [vp, vp, vp, vp, vp, lg]
        L.oracle_softmax_rows_bf16.argtypes = [vp, vp, lg, lg]
        L.oracle_normalize_rows_f32.argtypes = [vp, vp, lg, lg, ctypes.c_float]
        L.oracle_relu_scale_bias_f16.argtypes = [vp, vp, vp, vp, lg, lg, lg]
        L.oracle_channel_stats_f16.argtypes = [vp, vp, vp, lg, lg, lg]
        L.oracle_rows_f32.argtypes = [vp, vp, vp, vp, lg, lg]
        _lib = L
    return _lib


def dtype_size(dtype: int) -> int:
    return lib().oracle_dtype_size(dtype)


def convert(src: np.ndarray, src_dtype: int, dst_dtype: int, threads: int = 0) -> np.ndarray:
    """Out-of-place storage conversion of a flat/ND carrier array."""
    src = np.ascontiguousarray(src)
    assert src.dtype == np.dtype(CARRIER[src_dtype]), (src.dtype, src_dtype)
    dst = np.empty(src.shape, dtype=CARRIER[dst_dtype])
    rc = lib().oracle_convert(src.ctypes.data, dst.ctypes.data, src_dtype, dst_dtype, src.size, threads)
    if rc < 0:
        raise ValueError("oracle_convert: unsupported dtype pair")
    return dst


def convert_raw(src_ptr: int, dst_ptr: int, src_dtype: int, dst_dtype: int, n: int, threads: int = 0) -> int:
    """Pointer-level conversion (used for in-place checks and for the timed CPU baseline). Returns threads used."""
    return lib().oracle_convert(src_ptr, dst_ptr, src_dtype, dst_dtype, n, threads)


def to_f32(a: np.ndarray, dtype: int) -> np.ndarray:
    return convert(a, dtype, FP32) if dtype != FP32 else np.ascontiguousarray(a, dtype=np.float32)


def from_f32(a: np.ndarray, dtype: int) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    return convert(a, FP32, dtype) if dtype != FP32 else a


def round_through(a: np.ndarray, dtype: int) -> np.ndarray:
    """fp32 values rounded to `dtype` storage and widened back to fp32."""
    return to_f32(from_f32(a, dtype), dtype)


def _geom(arr: np.ndarray, axes):
    dims = (ctypes.c_uint64 * arr.ndim)(*arr.shape)
    item = arr.dtype.itemsize
    strides = (ctypes.c_uint64 * arr.ndim)(*[s // item for s in arr.strides])
    ax = (ctypes.c_uint32 * len(axes))(*axes)
    return dims, strides, ax


def _out_shape(arr: np.ndarray, axes):
    return [1 if i in axes else d for i, d in enumerate(arr.shape)]


def reduce(op: int, arr: np.ndarray, in_dtype: int, axes, out_dtype: int = FP32, scale: float = 1.0) -> np.ndarray:
    """fp32-accumulating reduction in row-major order of the reduced coordinates; keeps reduced axes as 1."""
    axes = sorted(int(a) for a in axes)
    dims, strides, ax = _geom(arr, axes)
    out = np.empty(_out_shape(arr, axes), dtype=CARRIER[out_dtype])
    rc = lib().oracle_reduce(op, arr.ctypes.data, in_dtype, dims, strides, arr.ndim, ax, len(axes), scale, out.ctypes.data, out_dtype)
    if rc:
        raise ValueError("oracle_reduce rejected the arguments")
    return out


def reduce_f64(op: int, arr: np.ndarray, in_dtype: int, axes) -> np.ndarray:
    axes = sorted(int(a) for a in axes)
    dims, strides, ax = _geom(arr, axes)
    out = np.empty(_out_shape(arr, axes), dtype=np.float64)
    rc = lib().oracle_reduce_f64(op, arr.ctypes.data, in_dtype, dims, strides, arr.ndim, ax, len(axes), out.ctypes.data)
    if rc:
        raise ValueError("oracle_reduce_f64 rejected the arguments")
    return out


def arg_reduce(op: int, arr: np.ndarray, in_dtype: int, axes):
    axes = sorted(int(a) for a in axes)
    dims, strides, ax = _geom(arr, axes)
    shape = _out_shape(arr, axes)
    idx = np.empty(shape, dtype=np.uint64)
    val = np.empty(shape, dtype=np.float32)
    rc = lib().oracle_arg_reduce(op, arr.ctypes.data, in_dtype, dims, strides, arr.ndim, ax, len(axes), idx.ctypes.data, val.ctypes.data)
    if rc:
        raise ValueError("oracle_arg_reduce rejected the arguments")
    return idx, val


# ---- BASELINE expression workloads on the host cores (thor_oracle_expr.c) ------------------------------------------------------
def _c(a, dtype):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.dtype(dtype), (a.dtype, dtype)
    return a


def expr_config1(a, b, c, d):
    """out = (a*b + c) * sigmoid(d) in fp32; returns (out, threads)."""
    a, b, c, d = (_c(v, np.float32) for v in (a, b, c, d))
    out = np.empty_like(a)
    threads = lib().oracle_expr_config1(a.ctypes.data, b.ctypes.data, c.ctypes.data, d.ctypes.data, out.ctypes.data, a.size)
    return out, threads


def softmax_rows_bf16(x_bits):
    x_bits = _c(x_bits, np.uint16)
    rows, cols = x_bits.shape
    out = np.empty((rows, cols), dtype=np.float32)
    threads = lib().oracle_softmax_rows_bf16(x_bits.ctypes.data, out.ctypes.data, rows, cols)
    return out, threads


def normalize_rows_f32(x, eps=1e-5):
    x = _c(x, np.float32)
    rows, cols = x.shape
    out = np.empty_like(x)
    threads = lib().oracle_normalize_rows_f32(x.ctypes.data, out.ctypes.data, rows, cols, eps)
    return out, threads


def relu_scale_bias_f16(x, scale, bias):
    """x: float16 [N,C,H,W]; scale, bias: float16 with C elements."""
    x, scale, bias = (_c(v, np.float16) for v in (x, scale, bias))
    n, c = x.shape[0], x.shape[1]
    hw = x.size // (n * c)
    out = np.empty_like(x)
    threads = lib().oracle_relu_scale_bias_f16(x.ctypes.data, scale.ctypes.data, bias.ctypes.data, out.ctypes.data, n, c, hw)
    return out, threads


def channel_stats_f16(x):
    x = _c(x, np.float16)
    n, c = x.shape[0], x.shape[1]
    hw = x.size // (n * c)
    total, squares = np.empty(c, np.float32), np.empty(c, np.float32)
    threads = lib().oracle_channel_stats_f16(x.ctypes.data, total.ctypes.data, squares.ctypes.data, n, c, hw)
    return total, squares, threads


def rows_f32(x):
    """row sums, row maxima and row argmax (uint32) of an fp32 matrix."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    s, m, a = np.empty(rows, np.float32), np.empty(rows, np.float32), np.empty(rows, np.uint32)
    threads = lib().oracle_rows_f32(x.ctypes.data, s.ctypes.data, m.ctypes.data, a.ctypes.data, rows, cols)
    return s, m, a, threads
