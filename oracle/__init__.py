"""ctypes front-end of the CPU oracle (test infrastructure only).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the product
(thor_amd) never does.  The arithmetic lives in thor_oracle.c; expression evaluation lives in expr.py.
"""
from __future__ import annotations

import ctypes
import math
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
    sources = [os.path.join(_HERE, name) for name in ("thor_oracle.c", "thor_oracle_expr.c", "thor_oracle_scan.c", "thor_oracle.h")]
    stale = (not os.path.exists(_LIB_PATH)) or any(os.path.getmtime(_LIB_PATH) < os.path.getmtime(src) for src in sources)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
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
        L.oracle_scan.argtypes = [vp, ctypes.c_int, lg, vp, lg, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp]
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


# ---- prefix scans --------------------------------------------------------------------------------------------------------------
SCAN_SUM, SCAN_MIN, SCAN_MAX, SCAN_PRODUCT, SCAN_ARGMIN, SCAN_ARGMAX = range(6)


def _scan_segment_fast(x, base, integer, dtype):
    """Inclusive forward scan of one segment with NumPy's sequential accumulate routines, for the cases where they perform the
    same operations in the same order as the element-by-element walk: returns (values, winner positions) or None."""
    if x.size == 0:
        return x.copy(), np.zeros(0, np.int64)
    if base in (SCAN_MIN, SCAN_MAX):
        if not integer and np.isnan(x).any():
            return None
        running = (np.minimum if base == SCAN_MIN else np.maximum).accumulate(x)
        changed = np.concatenate([[True], running[1:] != running[:-1]])  # a new running value is set by a strictly better element
        positions = np.maximum.accumulate(np.where(changed, np.arange(x.size), 0))
        return x[positions], positions  # the winner's own bits (-0.0 and +0.0 compare equal: the earlier one stays)
    if integer:
        if base == SCAN_SUM:
            return np.cumsum(x, dtype=np.uint64) & np.uint64(0xFFFFFFFF), None
        return None
    if dtype == FP32:
        return (np.cumsum(x, dtype=np.float32) if base == SCAN_SUM else np.cumprod(x, dtype=np.float32)), None
    if dtype == FP16:
        with np.errstate(over="ignore", invalid="ignore"):
            half = x.astype(np.float16)
            return (np.cumsum(half, dtype=np.float16) if base == SCAN_SUM else np.cumprod(half, dtype=np.float16)).astype(np.float32), None
    return None


def scan(values: np.ndarray, op: int, inclusive: bool = True, reverse: bool = False, segment_size: int = 0, offsets=None, dtype: int = FP32,
         fast: bool = True, engine: str = None):
    """Sequential restatement of the reference's scans over a flat array of `dtype` carriers
    (Utilities/TensorOperations/Cub/CubScan.cu:47-93 operators, :106-196 identities; CubSegmentedScan.cu for segments).

    Every combine rounds to the element type (16-bit floats add and multiply in fp32, then round); min / max keep the earlier
    element unless the later one is strictly smaller / larger; the first element of a segment is taken as it is.  Exclusive
    scans start with 0, 1, the largest / smallest value (+-inf for floats); arg scans return UINT32 flattened indices, with
    0xFFFFFFFF where the prefix is empty.  Segments: `segment_size` > 0 -> consecutive runs of that length; `offsets` -> the
    ranges [offsets[s], offsets[s + 1]); neither -> one scan.  Elements outside every segment keep 0.  `reverse` scans every
    segment from its end.  Value scans return carriers of `dtype`.

    Three engines perform the same walk and the tests hold them against each other: "c" (thor_oracle_scan.c, the default: fast
    enough for millions of elements in every dtype), "python" (the loop below; `fast=False` selects it) and "numpy" (NumPy's
    sequential accumulate routines where they do the same operations in the same order, the loop elsewhere)."""
    flat = np.ascontiguousarray(values).reshape(-1)
    n = flat.size
    arg = op in (SCAN_ARGMIN, SCAN_ARGMAX)
    base = {SCAN_ARGMIN: SCAN_MIN, SCAN_ARGMAX: SCAN_MAX}.get(op, op)
    integer = dtype == UINT32
    engine = engine or ("c" if fast else "python")
    if engine == "c":
        if offsets is not None:
            pairs = [(int(offsets[s]), int(offsets[s + 1])) for s in range(len(offsets) - 1)]
        elif segment_size:
            pairs = [(b, b + segment_size) for b in range(0, n, segment_size)]
        else:
            pairs = [(0, n)]
        table = np.ascontiguousarray(np.array(pairs, np.int64).reshape(-1))
        carrier = np.ascontiguousarray(flat, dtype=CARRIER[dtype])
        out_values = np.empty(n, CARRIER[dtype])
        out_index = np.empty(n, np.uint32)
        rc = lib().oracle_scan(carrier.ctypes.data, dtype, n, table.ctypes.data, len(pairs), base, int(bool(inclusive)), int(bool(reverse)),
                               None if arg else out_values.ctypes.data, out_index.ctypes.data if arg else None)
        if rc != 0:
            raise ValueError(f"oracle_scan failed with {rc}")
        return (out_index if arg else out_values).reshape(np.shape(values))
    fast = engine == "numpy"
    work = flat.astype(np.uint64) if integer else to_f32(flat, dtype).astype(np.float32)

    def rounded(x):
        if integer:
            return np.uint64(int(x) & 0xFFFFFFFF)
        return to_f32(from_f32(np.array([x], np.float32), dtype), dtype)[0]

    identity = {SCAN_SUM: 0, SCAN_PRODUCT: 1, SCAN_MIN: 0xFFFFFFFF if integer else np.inf, SCAN_MAX: 0 if integer else -np.inf}[base]
    if offsets is not None:
        bounds = [(int(offsets[s]), int(offsets[s + 1])) for s in range(len(offsets) - 1)]
    elif segment_size:
        bounds = [(b, b + segment_size) for b in range(0, n, segment_size)]
    else:
        bounds = [(0, n)]
    out_values = np.zeros(n, np.uint64 if integer else np.float32)
    out_index = np.zeros(n, np.uint32)
    with np.errstate(over="ignore", invalid="ignore"):
        for begin, end in bounds:
            quick = _scan_segment_fast(work[begin:end][::-1] if reverse else work[begin:end], base, integer, dtype) if fast else None
            if quick is not None and end > begin:
                running_values, positions = quick
                if positions is None:
                    positions = np.zeros(end - begin, np.int64)
                where = (end - 1 - positions) if reverse else (begin + positions)
                if not inclusive:
                    running_values = np.concatenate([[identity], running_values[:-1]]).astype(running_values.dtype)
                    where = np.concatenate([[0xFFFFFFFF], where[:-1]])
                target = slice(begin, end)
                out_values[target] = running_values[::-1] if reverse else running_values
                out_index[target] = (where[::-1] if reverse else where).astype(np.uint32)
                continue
            order = range(end - 1, begin - 1, -1) if reverse else range(begin, end)
            running, winner = None, 0xFFFFFFFF
            for i in order:
                x = work[i]
                if not inclusive:
                    out_values[i] = identity if running is None else running
                    out_index[i] = winner
                if running is None:
                    running, winner = x, i
                elif base == SCAN_SUM:
                    running = rounded(np.float32(running) + np.float32(x)) if not integer else rounded(int(running) + int(x))
                elif base == SCAN_PRODUCT:
                    running = rounded(np.float32(running) * np.float32(x)) if not integer else rounded(int(running) * int(x))
                elif (x < running) if base == SCAN_MIN else (running < x):
                    running, winner = x, i
                if inclusive:
                    out_values[i] = running
                    out_index[i] = winner
    if arg:
        return out_index.reshape(np.shape(values))
    if integer:
        return out_values.astype(np.uint32).reshape(np.shape(values))
    return from_f32(out_values.astype(np.float32), dtype).reshape(np.shape(values))


# ---- rotary position embedding -------------------------------------------------------------------------------------------
ROPE_NONE, ROPE_LINEAR, ROPE_DYNAMIC_NTK, ROPE_YARN, ROPE_LONGROPE, ROPE_LLAMA3 = 0, 1, 2, 3, 4, 5


def select_flagged(values: np.ndarray, flags: np.ndarray):
    """The elements of `values` whose flag is nonzero, in input order, and their number: what cub::DeviceSelect::Flagged
    documents and the reference relies on (Utilities/TensorOperations/Cub/CubSelect.cu:43-50; CUB is a third-party library
    that is not part of the reference tree).  Carriers pass through untouched."""
    flat = np.ascontiguousarray(values).reshape(-1)
    raised = np.ascontiguousarray(flags).reshape(-1) != 0
    kept = flat[raised[:flat.size]] if flat.size else flat[:0]
    return kept, int(kept.size)


def key_order_image(keys: np.ndarray, dtype: int) -> np.ndarray:
    """An int64 per key that sorts like the key does for the reference's selection library: integers by value, floats by sign
    and magnitude of their bits, so -0 sorts below +0 and NaNs beyond the infinities (the radix order cub documents for
    floating-point keys)."""
    flat = np.ascontiguousarray(keys).reshape(-1)
    if dtype in (UINT8, UINT16, UINT32, INT8, INT16, INT32):
        return flat.astype(np.int64)
    width = {FP16: 16, BF16: 16, FP32: 32}[dtype]
    bits = flat.view({16: np.uint16, 32: np.uint32}[width]).astype(np.int64)
    sign = 1 << (width - 1)
    magnitude = bits & (sign - 1)
    return np.where(bits & sign, -magnitude - 1, magnitude)


def top_k(keys: np.ndarray, k: int, largest: bool = True, dtype: int = FP32, segment_size: int = 0):
    """The k largest (or smallest) keys of the flat array, or of every run of `segment_size` keys, best first; k is capped at
    the run length (Utilities/TensorOperations/Cub/CubTopK.cu:27-60,333-420 device-wide, :120-330,520-735 fixed-size segments;
    the selection itself is cub's).  The reference's output is unordered and which of several equal keys is taken is not
    fixed, so callers compare sorted keys; returns (keys [segments, k] as carriers, positions [segments, k] of one valid
    choice, and the order image of the k-th key per segment, which decides whether a candidate answer is admissible)."""
    flat = np.ascontiguousarray(keys).reshape(-1)
    run = segment_size if segment_size else flat.size
    if run == 0:
        return flat[:0].reshape(0, 0), np.zeros((0, 0), np.int64), np.zeros((0,), np.int64)
    image = key_order_image(flat, dtype).reshape(-1, run)
    take = min(k, run)
    ranked = np.argsort(-image if largest else image, axis=1, kind="stable")[:, :take]
    positions = ranked + np.arange(image.shape[0])[:, None] * run
    chosen = flat[positions.reshape(-1)].reshape(image.shape[0], take)
    threshold = np.take_along_axis(image, ranked[:, take - 1:take], axis=1)[:, 0] if take else np.zeros((image.shape[0],), np.int64)
    return chosen, positions, threshold


def rope_attention_factor(scaling_kind=ROPE_NONE, scaling_factor=1.0, original_max_position_embeddings=0, attention_factor=None):
    """The magnitude correction a ROPE node carries (Utilities/Expression/Expression.cpp:4398-4413): the caller's, else
    0.1 ln(s) + 1 for YaRN and sqrt(1 + ln(s) / ln(original_max)) for LongRoPE when s > 1, else 1."""
    if attention_factor is not None:
        return float(attention_factor)
    if scaling_kind == ROPE_YARN:
        return 1.0 if scaling_factor <= 1.0 else 0.1 * math.log(scaling_factor) + 1.0
    if scaling_kind == ROPE_LONGROPE:
        return 1.0 if scaling_factor <= 1.0 else math.sqrt(1.0 + math.log(scaling_factor) / math.log(float(original_max_position_embeddings)))
    return 1.0


def rope_frequencies(rotary_dim, base=10000.0, scaling_kind=ROPE_NONE, scaling_factor=1.0, original_max_position_embeddings=0,
                     yarn_beta_fast=32.0, yarn_beta_slow=1.0, llama3_low_freq_factor=1.0, llama3_high_freq_factor=4.0,
                     long_rope_short_factors=None, long_rope_long_factors=None, sequence_length=1.0):
    """fp32 frequency of every pair, operation by operation as the generated kernel of the reference computes it
    (Utilities/Expression/CudaSourceEmitter.cpp:3607-3690).  `sequence_length` is max(effective length + max(offset, 0), 1),
    which only the Dynamic-NTK and LongRoPE rules read.  Linear scaling leaves the frequencies alone (it divides the position)."""
    f = np.float32
    pairs = np.arange(rotary_dim // 2, dtype=np.float32)
    rot = f(rotary_dim)
    b = f(base)
    s = f(scaling_factor)
    original = f(original_max_position_embeddings)
    seq_len = f(sequence_length)
    if scaling_kind == ROPE_DYNAMIC_NTK:
        if seq_len > original and rotary_dim > 2:
            ratio = f(f(f(s * seq_len) / original) - f(s - f(1.0)))
            b = f(b * np.power(ratio, f(rot / f(rotary_dim - 2)), dtype=np.float32))
        return np.power(b, (f(-2.0) * pairs) / rot, dtype=np.float32)
    if scaling_kind == ROPE_YARN:
        pos_freq = np.power(b, (f(2.0) * pairs) / rot, dtype=np.float32)
        extrapolated = f(1.0) / pos_freq
        interpolated = f(1.0) / (s * pos_freq)
        log_base = np.log(b, dtype=np.float32)
        two_pi = f(6.2831853071795864769)
        low = f(rot * np.log(f(original / f(f(yarn_beta_fast) * two_pi)), dtype=np.float32)) / f(f(2.0) * log_base)
        high = f(rot * np.log(f(original / f(f(yarn_beta_slow) * two_pi)), dtype=np.float32)) / f(f(2.0) * log_base)
        low = max(f(np.floor(low)), f(0.0))
        high = min(f(np.ceil(high)), f(rotary_dim - 1))
        if low == high:
            high = f(high + f(0.001))
        ramp = np.minimum(np.maximum((pairs - low) / f(high - low), f(0.0)), f(1.0)).astype(np.float32)
        return (interpolated * ramp + extrapolated * (f(1.0) - ramp)).astype(np.float32)
    if scaling_kind == ROPE_LONGROPE:
        stretch = np.asarray(long_rope_long_factors if seq_len > original else long_rope_short_factors, dtype=np.float32)
        return (f(1.0) / (stretch * np.power(b, (f(2.0) * pairs) / rot, dtype=np.float32))).astype(np.float32)
    plain = np.power(b, (f(-2.0) * pairs) / rot, dtype=np.float32)
    if scaling_kind == ROPE_LLAMA3:
        two_pi = f(6.2831853071795864769)
        wavelength = two_pi / plain
        low_wavelength = f(original / f(llama3_low_freq_factor))
        high_wavelength = f(original / f(llama3_high_freq_factor))
        smooth = (original / wavelength - f(llama3_low_freq_factor)) / f(f(llama3_high_freq_factor) - f(llama3_low_freq_factor))
        blended = (f(1.0) - smooth) * (plain / s) + smooth * plain
        return np.where(wavelength > low_wavelength, plain / s, np.where(wavelength < high_wavelength, plain, blended)).astype(np.float32)
    return plain


def rope(x: np.ndarray, dtype: int = FP32, *, sequence_axis=2, head_dim_axis=3, rotary_dim=0, base=10000.0, position_offset=0, interleaved=False,
         inverse=False, scaling_kind=ROPE_NONE, scaling_factor=1.0, original_max_position_embeddings=0, attention_factor=None, yarn_beta_fast=32.0,
         yarn_beta_slow=1.0, llama3_low_freq_factor=1.0, llama3_high_freq_factor=4.0, long_rope_short_factors=None, long_rope_long_factors=None,
         position_ids=None, effective_sequence_length=None, out_dtype=None):
    """Rotary position embedding of carriers `x` of `dtype`, in fp32, restating the reference's generated kernel
    (Utilities/Expression/CudaSourceEmitter.cpp:3538-3697): the first element a and second element b of pair j at position p
    become a cos(t) - b sin(t) and a sin(t) + b cos(t), t = p * frequency(j), sine and cosine scaled by the attention factor and
    the sine negated for the inverse; p = coordinate + offset (divided by the factor for linear scaling) or the given position
    ids; the pairs are (j, j + rotary/2), or (2j, 2j + 1) when interleaved; coordinates of the head dimension beyond rotary_dim
    pass through.  Returns carriers of `out_dtype` (default: `dtype`)."""
    out_dtype = dtype if out_dtype is None else out_dtype
    f = np.float32
    values = to_f32(np.ascontiguousarray(x).reshape(-1), dtype).astype(np.float32).reshape(np.shape(x))
    moved = np.moveaxis(values, (sequence_axis, head_dim_axis), (-2, -1))  # [..., S, D] view
    seq, head_dim = moved.shape[-2], moved.shape[-1]
    rotary = head_dim if rotary_dim == 0 else rotary_dim
    assert 0 < rotary <= head_dim and rotary % 2 == 0
    half = rotary // 2
    if position_ids is not None:
        positions = np.asarray(position_ids).reshape(-1).astype(np.float32)
        assert position_offset == 0 and positions.size == seq
    else:
        positions = np.arange(seq, dtype=np.float32) + f(position_offset)
    if scaling_kind == ROPE_LINEAR:
        positions = positions / f(scaling_factor)
    extent = f(seq) if effective_sequence_length is None else f(effective_sequence_length)
    seq_len = max(f(extent + f(max(0, position_offset))), f(1.0))
    freq = rope_frequencies(rotary, base, scaling_kind, scaling_factor, original_max_position_embeddings, yarn_beta_fast, yarn_beta_slow,
                            llama3_low_freq_factor, llama3_high_freq_factor, long_rope_short_factors, long_rope_long_factors, seq_len)
    theta = (positions[:, None] * freq[None, :]).astype(np.float32)
    # sine and cosine of the fp32 angle, correctly rounded to fp32 (device libraries stay within 2 ulp of this)
    sn = np.sin(theta.astype(np.float64)).astype(np.float32)
    cs = np.cos(theta.astype(np.float64)).astype(np.float32)
    factor = rope_attention_factor(scaling_kind, scaling_factor, original_max_position_embeddings, attention_factor)
    if factor != 1.0:
        sn, cs = sn * f(factor), cs * f(factor)
    if inverse:
        sn = -sn
    first = np.arange(0, rotary, 2) if interleaved else np.arange(half)
    second = first + 1 if interleaved else first + half
    a, b = moved[..., first], moved[..., second]
    result = moved.copy()
    result[..., first] = a * cs - b * sn
    result[..., second] = a * sn + b * cs
    result = np.moveaxis(result, (-2, -1), (sequence_axis, head_dim_axis))
    return from_f32(np.ascontiguousarray(result, dtype=np.float32).reshape(-1), out_dtype).reshape(np.shape(x))
