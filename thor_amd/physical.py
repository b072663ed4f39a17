"""Python mirror of the reference's `thor.physical` surface for the hot path -- Expression, FusedEquation ("compile"),
Equation (the stamped plan), PhysicalTensor, Stream, Placement -- bound to libthor_amd.so through include/thor_c_api.h.

The shapes of the calls follow bindings/python/src/core/physical/expression.cpp:602-2866 of the reference so that its
test helpers (`_copy_numpy_to_gpu`, `_run_expr`, `_run_staged_expr`) read the same here.  Nothing is computed in Python.
"""
from __future__ import annotations

import ctypes
import enum
from typing import Dict, Iterable, List, Optional, Sequence, Union

import numpy as np

from . import _lib
from .dtypes import DataType, numpy_carrier

_vp, _i, _u64, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_size_t
_u64p = ctypes.POINTER(ctypes.c_uint64)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_cp = ctypes.c_char_p
_cpp = ctypes.POINTER(ctypes.c_char_p)
_vpp = ctypes.POINTER(ctypes.c_void_p)
_fp = ctypes.POINTER(ctypes.c_float)
UINT64_MAX = (1 << 64) - 1


class ReductionGeometry(ctypes.Structure):
    _fields_ = [
        ("path", _i), ("reduced_axes_are_contiguous", _i),
        ("outer_size", _u64), ("reduction_size", _u64), ("inner_size", _u64),
        ("input_elements", _u64), ("output_elements", _u64),
        ("rank", _i), ("output_dimensions", _u64 * 16),
        ("squeezed_rank", _i), ("squeezed_output_dimensions", _u64 * 16),
        ("device_transform_uses_affine_stride", _i), ("affine_input_stride", _u64),
    ]


PROTOTYPES = {
    "thor_last_error": (_cp, []),
    "thor_stream_create": (_vp, [_i]), "thor_stream_destroy": (None, [_vp]), "thor_stream_synchronize": (_i, [_vp]),
    "thor_stream_raw": (_vp, [_vp]), "thor_stream_gpu_num": (_i, [_vp]),
    "thor_tensor_create": (_vp, [_i, _i, _i, _u64p, _i]), "thor_tensor_clone_handle": (_vp, [_vp]), "thor_tensor_destroy": (None, [_vp]),
    "thor_tensor_mem_ptr": (_vp, [_vp]), "thor_tensor_dtype": (_i, [_vp]), "thor_tensor_rank": (_i, [_vp]),
    "thor_tensor_dims": (_i, [_vp, _u64p]), "thor_tensor_strides": (_i, [_vp, _u64p]), "thor_tensor_num_elements": (_u64, [_vp]),
    "thor_tensor_device_type": (_i, [_vp]), "thor_tensor_device_num": (_i, [_vp]), "thor_tensor_is_dense": (_i, [_vp]),
    "thor_tensor_copy_from_async": (_i, [_vp, _vp, _vp]), "thor_tensor_memset_async": (_i, [_vp, _i, _vp]),
    "thor_tensor_reshape": (_i, [_vp, _u64p, _i]), "thor_tensor_alias_view": (_vp, [_vp, _u64p, _u64p, _i, _u64]),
    "thor_convert_type": (_i, [_vp, _vp, _i, _i, ctypes.c_int64, _vp, _i]),
    "thor_convert_type_cpu": (_i, [_vp, _vp, _i, _i, ctypes.c_int64]),
    "thor_reduction_analyze_geometry": (_i, [_u64p, _u64p, _i, _u32p, _i, ctypes.POINTER(ReductionGeometry)]),
    "thor_reduction_map_index": (_i, [_u64p, _u64p, _i, _u32p, _i, _u64, _u64, _u64p]),
    "thor_reduction_stamp": (_vp, [_i, _u32p, _i, _i, ctypes.c_float, _vp, _vp, _vp]),
    "thor_stamped_reduction_destroy": (None, [_vp]), "thor_stamped_reduction_run": (_i, [_vp]),
    "thor_stamped_reduction_run_scaled": (_i, [_vp, ctypes.c_float]), "thor_stamped_reduction_run_on": (_i, [_vp, _vp]),
    "thor_stamped_reduction_output": (_vp, [_vp]), "thor_stamped_reduction_path": (_i, [_vp]),
    "thor_stamped_reduction_workspace_bytes": (_sz, [_vp]), "thor_stamped_reduction_variant": (_i, [_vp, _cp, _sz]),
    "thor_stamped_arg_reduction_variant": (_i, [_vp, _cp, _sz]),
    "thor_segmented_reduction_stamp": (_vp, [_i, _i, _i, _vp, _vp, _vp, _i, _vp]),
    "thor_stamped_segmented_reduction_destroy": (None, [_vp]), "thor_stamped_segmented_reduction_run": (_i, [_vp]),
    "thor_stamped_segmented_reduction_output": (_vp, [_vp]), "thor_stamped_segmented_reduction_workspace_bytes": (_sz, [_vp]),
    "thor_stamped_segmented_reduction_variant": (_i, [_vp, _cp, _sz]),
    "thor_segmented_broadcast": (_i, [_vp, _vp, _vp, _i, _vp]),
    "thor_scan": (_i, [_vp, _vp, _vp, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, _i, _i, _i, _i, _vp, _cp, _sz]),
    "thor_scan_waits_recovered": (ctypes.c_uint64, []),
    "thor_scan_no_alloc": (_i, [_vp, _vp, _vp, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, _i, _i, _i, _i, _vp, _cp, _sz]),
    "thor_select_flagged": (_i, [_vp, _vp, _vp, _vp, ctypes.c_uint64, _vp, _cp, _sz]),
    "thor_select_flagged_prepare": (_vp, [_vp, _vp, _vp, _vp, ctypes.c_uint64]),
    "thor_topk_prepare": (_vp, [_vp, _vp, _vp, _vp, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, _i, _i]),
    "thor_selection_plan_temp_bytes": (_sz, [_vp]), "thor_selection_plan_run": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "thor_selection_plan_variant": (_i, [_vp, _cp, _sz]), "thor_selection_plan_destroy": (None, [_vp]),
    "thor_topk": (_i, [_vp, _vp, _vp, _vp, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, _i, _i, _vp, _cp, _sz]),
    "thor_reduction_generate_source": (_i, [_i, _i, _i, _i, _i, _u64p, _u64p, _i, _u32p, _i, _cp, _sz, ctypes.POINTER(_sz)]),
    "thor_arg_reduction_stamp": (_vp, [_i, _u32p, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "thor_stamped_arg_reduction_destroy": (None, [_vp]), "thor_stamped_arg_reduction_run": (_i, [_vp]),
    "thor_stamped_arg_reduction_value_output": (_vp, [_vp]), "thor_stamped_arg_reduction_index_output": (_vp, [_vp]),
    "thor_stamped_arg_reduction_path": (_i, [_vp]),
    "thor_expr_input": (_vp, [_cp, _i, _i]), "thor_expr_runtime_scalar": (_vp, [_cp, _i, _i]), "thor_expr_scalar": (_vp, [ctypes.c_double]),
    "thor_expr_fill": (_vp, [ctypes.c_double, _u64p, _i, _i]), "thor_expr_binary": (_vp, [_cp, _vp, _vp]),
    "thor_expr_ragged": (_vp, [_cp, _vp, _vp, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64]), "thor_expr_unary": (_vp, [_cp, _vp]),
    "thor_expr_unary_params": (_vp, [_cp, _vp, ctypes.c_double, ctypes.c_double]), "thor_expr_where": (_vp, [_vp, _vp, _vp]),
    "thor_expr_cast": (_vp, [_vp, _i]), "thor_expr_with_dtypes": (_vp, [_vp, _i, _i]),
    "thor_expr_reduce": (_vp, [_cp, _vp, _u64p, _i, _u64p, _i]), "thor_expr_reshape": (_vp, [_vp, _u64p, _i]),
    "thor_expr_strided_view": (_vp, [_vp, _u64p, _u64p, _i, ctypes.c_uint64]),
    "thor_expr_take_along_axis": (_vp, [_vp, _vp, ctypes.c_int64]),
    "thor_expr_rope": (_vp, [_vp, _vp, _vp, _vp]),
    "thor_expr_scan": (_vp, [_vp, _vp, _i, ctypes.c_int64, _i, _i]),
    "thor_expr_unsqueeze": (_vp, [_vp, _u64p, _i]), "thor_expr_squeeze": (_vp, [_vp, _u64p, _i]), "thor_expr_destroy": (None, [_vp]),
    "thor_expr_num_nodes": (_i, [_vp]), "thor_expr_canonical": (_i, [_vp, _cp, _sz, ctypes.POINTER(_sz)]),
    "thor_outputs_create": (_vp, [_cpp, _vpp, _i]), "thor_outputs_destroy": (None, [_vp]),
    "thor_outputs_conditional": (_vp, [_vp, _vp, _vpp, _vpp, _i, _vp]),
    "thor_fused_equation_compile": (_vp, [_vp, _i]), "thor_fused_equation_destroy": (None, [_vp]),
    "thor_fused_equation_compile_backward": (_vp, [_vp, _cpp, _i, _cpp, _cpp, _i, _i]),
    "thor_fused_equation_num_outputs": (_i, [_vp]), "thor_fused_equation_output_name": (_i, [_vp, _i, _cp, _sz]),
    "thor_fused_equation_stamp": (_vp, [_vp, _cpp, _vpp, _i, _cpp, _vpp, _i, _vp]),
    "thor_fused_equation_stamp_with_tensor_scalars": (_vp, [_vp, _cpp, _vpp, _i, _cpp, _vpp, _u64p, ctypes.POINTER(_i), _i, _cpp, _vpp, _i, _vp]),
    "thor_expr_tensor_runtime_scalar": (_vp, [_cp, _i, _i]),
    "thor_fused_equation_run": (_i, [_vp, _cpp, _vpp, _i, _cpp, _fp, _i, _cpp, _vpp, _i, _vp]),
    "thor_fused_equation_output_shape": (_i, [_vp, _cpp, _vpp, _i, _cp, _u64p, ctypes.POINTER(_i), ctypes.POINTER(_i)]),
    "thor_plan_destroy": (None, [_vp]), "thor_plan_run": (_i, [_vp]), "thor_plan_run_with_scalars": (_i, [_vp, _cpp, _fp, _i]),
    "thor_plan_run_on": (_i, [_vp, _vp]), "thor_plan_output": (_vp, [_vp, _cp]), "thor_plan_num_stages": (_i, [_vp]),
    "thor_plan_stage_kind": (_i, [_vp, _i, _cp, _sz]), "thor_plan_stage_source": (_i, [_vp, _i, _cp, _sz, ctypes.POINTER(_sz)]),
    "thor_plan_stage_description": (_i, [_vp, _i, _cp, _sz]), "thor_plan_flop_count": (_u64, [_vp]),
    "thor_compiled_kernel_count": (_u64, []),
}

_bound = None


def lib():
    global _bound
    if _bound is None:
        L = _lib.load()
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _bound = L
    return _bound


_ERROR_TYPES = {"invalid_argument": ValueError, "out_of_range": IndexError, "logic_error": AssertionError}


def _raise_last(what: str):
    msg = (lib().thor_last_error() or b"").decode("utf-8", "replace")
    kind, _, text = msg.partition(": ")
    raise _ERROR_TYPES.get(kind, RuntimeError)(f"{what}: {text or msg}")


def _check(rc: int, what: str):
    if rc != 0:
        _raise_last(what)


def _handle(ptr, what: str):
    if not ptr:
        _raise_last(what)
    return ptr


def _u64_array(values: Sequence[int]):
    values = [int(v) for v in values]
    return (ctypes.c_uint64 * max(1, len(values)))(*values), len(values)


def _u32_array(values: Sequence[int]):
    values = [int(v) for v in values]
    return (ctypes.c_uint32 * max(1, len(values)))(*values), len(values)


def _names(names: Sequence[str]):
    return (ctypes.c_char_p * max(1, len(names)))(*[n.encode() for n in names])


def _ptrs(handles: Sequence[int]):
    return (ctypes.c_void_p * max(1, len(handles)))(*handles)


def _dtype_code(dtype: Optional[DataType]) -> int:
    return -1 if dtype is None else int(dtype)


class DeviceType(enum.IntEnum):
    cpu = 1
    gpu = 2


class Placement:
    def __init__(self, device_type: DeviceType, device_num: int = 0):
        self.device_type = DeviceType(device_type)
        self.device_num = device_num

    def __eq__(self, other):
        return isinstance(other, Placement) and (self.device_type, self.device_num) == (other.device_type, other.device_num)

    def __repr__(self):
        return "CPU" if self.device_type == DeviceType.cpu else f"GPU:{self.device_num}"


class Stream:
    """Stream(gpu_num): shared handle of one HIP stream (Utilities/Common/Stream.h:35-116)."""

    def __init__(self, gpu_num: int = 0):
        self._h = _handle(lib().thor_stream_create(gpu_num), "Stream")
        self.gpu_num = gpu_num

    @property
    def handle(self):  # raw hipStream_t, accepted by thor_amd.runtime helpers
        return lib().thor_stream_raw(self._h)

    def synchronize(self):
        _check(lib().thor_stream_synchronize(self._h), "Stream.synchronize")

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_stream_destroy(self._h)
                self._h = None
        except Exception:
            pass


class PhysicalTensor:
    class Descriptor:
        def __init__(self, dtype: DataType, dimensions: Sequence[int]):
            self.dtype = DataType(dtype)
            self.dimensions = [int(d) for d in dimensions]

        def get_dimensions(self) -> List[int]:
            return list(self.dimensions)

        def get_data_type(self) -> DataType:
            return self.dtype

    def __init__(self, placement: Placement, descriptor: "PhysicalTensor.Descriptor", _handle_ptr=None):
        if _handle_ptr is not None:
            self._h = _handle_ptr
        else:
            dims, rank = _u64_array(descriptor.dimensions)
            self._h = _handle(lib().thor_tensor_create(int(placement.device_type), placement.device_num, int(descriptor.dtype), dims, rank),
                              "PhysicalTensor")

    @classmethod
    def _wrap(cls, ptr) -> "PhysicalTensor":
        return cls(None, None, _handle_ptr=_handle(ptr, "tensor handle"))

    def get_descriptor(self) -> "PhysicalTensor.Descriptor":
        return PhysicalTensor.Descriptor(self.get_data_type(), self.get_dimensions())

    def get_data_type(self) -> DataType:
        return DataType(lib().thor_tensor_dtype(self._h))

    def get_dimensions(self) -> List[int]:
        rank = lib().thor_tensor_rank(self._h)
        out = (ctypes.c_uint64 * rank)()
        _check(lib().thor_tensor_dims(self._h, out), "get_dimensions")
        return list(out)

    def get_strides_elements(self) -> List[int]:
        rank = lib().thor_tensor_rank(self._h)
        out = (ctypes.c_uint64 * rank)()
        _check(lib().thor_tensor_strides(self._h, out), "get_strides_elements")
        return list(out)

    def get_placement(self) -> Placement:
        return Placement(DeviceType(lib().thor_tensor_device_type(self._h)), lib().thor_tensor_device_num(self._h))

    def get_total_num_elements(self) -> int:
        return lib().thor_tensor_num_elements(self._h)

    def is_dense_contiguous(self) -> bool:
        return bool(lib().thor_tensor_is_dense(self._h))

    def mem_ptr(self) -> int:
        return lib().thor_tensor_mem_ptr(self._h) or 0

    def numpy(self) -> np.ndarray:
        """Zero-copy view of a CPU tensor in its numpy carrier dtype (bf16 / fp8 appear as raw unsigned integers)."""
        if self.get_placement().device_type != DeviceType.cpu:
            raise RuntimeError("numpy() is only available for CPU tensors")
        if not self.is_dense_contiguous():
            raise RuntimeError("numpy() requires a dense tensor")
        carrier = numpy_carrier(self.get_data_type())
        n = self.get_total_num_elements()
        buf = (ctypes.c_char * (n * carrier.itemsize)).from_address(self.mem_ptr())
        arr = np.frombuffer(buf, dtype=carrier, count=n).reshape(self.get_dimensions())
        arr.flags.writeable = True
        buf._tensor = self  # the array's base is `buf`: it keeps this tensor, and with it the pinned memory, alive as long as the array lives
        return arr

    def copy_from_async(self, source: "PhysicalTensor", stream: Stream):
        _check(lib().thor_tensor_copy_from_async(self._h, source._h, stream._h), "copy_from_async")

    def memset_async(self, value: int, stream: Stream):
        _check(lib().thor_tensor_memset_async(self._h, value, stream._h), "memset_async")

    def reshape(self, dimensions: Sequence[int]):
        dims, rank = _u64_array(dimensions)
        _check(lib().thor_tensor_reshape(self._h, dims, rank), "reshape")

    def alias_view(self, dimensions: Sequence[int], strides_elements: Sequence[int], element_offset: int = 0) -> "PhysicalTensor":
        dims, rank = _u64_array(dimensions)
        strides, _ = _u64_array(strides_elements)
        return PhysicalTensor._wrap(lib().thor_tensor_alias_view(self._h, dims, strides, rank, element_offset))

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_tensor_destroy(self._h)
                self._h = None
        except Exception:
            pass


def convert_type_cpu(values: np.ndarray, source_dtype: DataType, dest_dtype: DataType) -> np.ndarray:
    """TypeConverter's host path (TypeConverter::cpuConvertTypeImpl) on a numpy carrier array."""
    values = np.ascontiguousarray(values)
    assert values.dtype == numpy_carrier(source_dtype)
    out = np.empty(values.shape, dtype=numpy_carrier(dest_dtype))
    _check(lib().thor_convert_type_cpu(values.ctypes.data, out.ctypes.data, int(source_dtype), int(dest_dtype), values.size), "convert_type_cpu")
    return out


# ---- reductions ------------------------------------------------------------------------------------------------------------
class CubReductionOp(enum.IntEnum):
    Sum = 0
    Min = 1
    Max = 2
    Product = 3
    Mean = 4
    L1Norm = 5
    L2Norm = 6


class CubArgReductionOp(enum.IntEnum):
    ArgMin = 0
    ArgMax = 1


class CubReductionPath(enum.IntEnum):
    DeviceTransformReduce = 0
    ContiguousFixedSegment = 1
    TiledFixedSegment = 2
    StridedFixedSegment = 3
    OffsetSegmented = 4


def analyze_geometry(dims: Sequence[int], axes: Union[int, Sequence[int]], strides: Optional[Sequence[int]] = None) -> ReductionGeometry:
    axes = [axes] if isinstance(axes, int) else list(axes)
    d, rank = _u64_array(dims)
    a, na = _u32_array(axes)
    s = _u64_array(strides)[0] if strides is not None else None
    out = ReductionGeometry()
    _check(lib().thor_reduction_analyze_geometry(d, s, len(dims), a, na, ctypes.byref(out)), "analyzeGeometry")
    return out


def map_logical_reduction_index(dims, axes, output_index, reduction_index, strides=None) -> int:
    d, _ = _u64_array(dims)
    a, na = _u32_array(axes)
    s = _u64_array(strides)[0] if strides is not None else None
    out = ctypes.c_uint64()
    _check(lib().thor_reduction_map_index(d, s, len(dims), a, na, output_index, reduction_index, ctypes.byref(out)), "mapLogicalReductionIndex")
    return out.value


def reduction_source(is_arg: bool, op: int, input_dtype: DataType, output_dtype: DataType, dims, axes, strides=None,
                     index_dtype: DataType = DataType.uint32) -> str:
    d, _ = _u64_array(dims)
    a, na = _u32_array(axes)
    s = _u64_array(strides)[0] if strides is not None else None
    cap = 1 << 20
    buf = ctypes.create_string_buffer(cap)
    need = ctypes.c_size_t()
    _check(lib().thor_reduction_generate_source(int(is_arg), int(op), int(input_dtype), int(output_dtype), int(index_dtype), d, s, len(dims), a, na,
                                                buf, cap, ctypes.byref(need)), "reduction_source")
    return buf.value.decode()


class StampedCubReduction:
    def __init__(self, ptr):
        self._h = ptr

    def run(self, output_scale: Optional[float] = None):
        if output_scale is None:
            _check(lib().thor_stamped_reduction_run(self._h), "StampedCubReduction.run")
        else:
            _check(lib().thor_stamped_reduction_run_scaled(self._h, output_scale), "StampedCubReduction.run")

    def run_on(self, stream: Stream):
        _check(lib().thor_stamped_reduction_run_on(self._h, stream._h), "StampedCubReduction.runOn")

    def get_output_tensor(self) -> PhysicalTensor:
        return PhysicalTensor._wrap(lib().thor_stamped_reduction_output(self._h))

    def get_path(self) -> CubReductionPath:
        return CubReductionPath(lib().thor_stamped_reduction_path(self._h))

    def get_workspace_size_in_bytes(self) -> int:
        return lib().thor_stamped_reduction_workspace_bytes(self._h)

    def get_kernel_variant(self) -> str:
        buf = ctypes.create_string_buffer(512)
        _check(lib().thor_stamped_reduction_variant(self._h, buf, 512), "variant")
        return buf.value.decode()

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_stamped_reduction_destroy(self._h)
                self._h = None
        except Exception:
            pass


class CubReduction:
    """CubReduction(op, axes, output_dtype=None, output_scale=1.0).stamp(input, stream[, preallocated_output])."""

    def __init__(self, op: CubReductionOp, axes: Union[int, Sequence[int]], output_dtype: Optional[DataType] = None, output_scale: float = 1.0):
        self.op, self.axes = int(op), ([axes] if isinstance(axes, int) else list(axes))
        self.output_dtype, self.output_scale = output_dtype, float(output_scale)

    def stamp(self, input: PhysicalTensor, stream: Stream, preallocated_output: Optional[PhysicalTensor] = None) -> StampedCubReduction:
        a, na = _u32_array(self.axes)
        ptr = lib().thor_reduction_stamp(self.op, a, na, _dtype_code(self.output_dtype), self.output_scale, input._h,
                                         preallocated_output._h if preallocated_output else None, stream._h)
        return StampedCubReduction(_handle(ptr, "CubReduction.stamp"))


class StampedCubArgReduction:
    def __init__(self, ptr):
        self._h = ptr

    def run(self):
        _check(lib().thor_stamped_arg_reduction_run(self._h), "StampedCubArgReduction.run")

    def get_value_output_tensor(self) -> Optional[PhysicalTensor]:
        ptr = lib().thor_stamped_arg_reduction_value_output(self._h)
        return PhysicalTensor._wrap(ptr) if ptr else None

    def get_index_output_tensor(self) -> Optional[PhysicalTensor]:
        ptr = lib().thor_stamped_arg_reduction_index_output(self._h)
        return PhysicalTensor._wrap(ptr) if ptr else None

    def get_path(self) -> CubReductionPath:
        return CubReductionPath(lib().thor_stamped_arg_reduction_path(self._h))

    def get_kernel_variant(self) -> str:
        buf = ctypes.create_string_buffer(512)
        _check(lib().thor_stamped_arg_reduction_variant(self._h, buf, 512), "variant")
        return buf.value.decode()

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_stamped_arg_reduction_destroy(self._h)
                self._h = None
        except Exception:
            pass


class CubArgReduction:
    def __init__(self, op: CubArgReductionOp, axes: Union[int, Sequence[int]], produce_value: bool = True, produce_index: bool = True,
                 value_output_dtype: Optional[DataType] = None, index_output_dtype: DataType = DataType.uint32):
        self.op, self.axes = int(op), ([axes] if isinstance(axes, int) else list(axes))
        self.produce_value, self.produce_index = produce_value, produce_index
        self.value_output_dtype, self.index_output_dtype = value_output_dtype, index_output_dtype

    def stamp(self, input: PhysicalTensor, stream: Stream, preallocated_value: Optional[PhysicalTensor] = None,
              preallocated_index: Optional[PhysicalTensor] = None) -> StampedCubArgReduction:
        a, na = _u32_array(self.axes)
        ptr = lib().thor_arg_reduction_stamp(self.op, a, na, int(self.produce_value), int(self.produce_index), _dtype_code(self.value_output_dtype),
                                             int(self.index_output_dtype), input._h, preallocated_value._h if preallocated_value else None,
                                             preallocated_index._h if preallocated_index else None, stream._h)
        return StampedCubArgReduction(_handle(ptr, "CubArgReduction.stamp"))


class StampedCubSegmentedReduction:
    def __init__(self, ptr):
        self._h = ptr

    def run(self):
        _check(lib().thor_stamped_segmented_reduction_run(self._h), "StampedCubSegmentedReduction.run")

    def get_output_tensor(self) -> PhysicalTensor:
        return PhysicalTensor._wrap(_handle(lib().thor_stamped_segmented_reduction_output(self._h), "getOutputTensor"))

    get_index_output_tensor = get_output_tensor

    def get_path(self) -> CubReductionPath:
        return CubReductionPath.OffsetSegmented

    def get_workspace_size_in_bytes(self) -> int:
        return lib().thor_stamped_segmented_reduction_workspace_bytes(self._h)

    def get_kernel_variant(self) -> str:
        buf = ctypes.create_string_buffer(512)
        _check(lib().thor_stamped_segmented_reduction_variant(self._h, buf, 512), "variant")
        return buf.value.decode()

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_stamped_segmented_reduction_destroy(self._h)
                self._h = None
        except Exception:
            pass


class CubSegmentedReduction:
    """Values [N, D...] reduced over the row ranges [offsets[i], offsets[i+1]) -> [B, D...] (sum, mean, min, max)."""

    def __init__(self, op: CubReductionOp, output_dtype: Optional[DataType] = None):
        self.op, self.output_dtype = op, output_dtype

    def _stamp(self, input, offsets, stream, preallocated, runtime):
        ptr = lib().thor_segmented_reduction_stamp(0, int(self.op), -1 if self.output_dtype is None else int(self.output_dtype), input._h, offsets._h,
                                                   preallocated._h if preallocated is not None else None, 1 if runtime else 0, stream._h)
        return StampedCubSegmentedReduction(_handle(ptr, "CubSegmentedReduction.stamp"))

    def stamp(self, input: PhysicalTensor, segment_offsets: PhysicalTensor, stream: Stream, preallocated_output: Optional[PhysicalTensor] = None):
        return self._stamp(input, segment_offsets, stream, preallocated_output, False)

    def stamp_runtime_offsets(self, input: PhysicalTensor, preallocated_output: PhysicalTensor, segment_offsets: PhysicalTensor, stream: Stream):
        return self._stamp(input, segment_offsets, stream, preallocated_output, True)


class CubSegmentedArgReduction:
    """Winner indices (packed row * D + d) of argmin / argmax over the same row ranges; empty segments give the all-ones index."""

    def __init__(self, op: CubArgReductionOp, index_output_dtype: DataType = DataType.uint64):
        self.op, self.index_output_dtype = op, index_output_dtype

    def _stamp(self, input, offsets, stream, preallocated, runtime):
        ptr = lib().thor_segmented_reduction_stamp(1, int(self.op), int(self.index_output_dtype), input._h, offsets._h,
                                                   preallocated._h if preallocated is not None else None, 1 if runtime else 0, stream._h)
        return StampedCubSegmentedReduction(_handle(ptr, "CubSegmentedArgReduction.stamp"))

    def stamp(self, input: PhysicalTensor, segment_offsets: PhysicalTensor, stream: Stream, preallocated_index_output: Optional[PhysicalTensor] = None):
        return self._stamp(input, segment_offsets, stream, preallocated_index_output, False)

    def stamp_runtime_offsets(self, input: PhysicalTensor, preallocated_index_output: PhysicalTensor, segment_offsets: PhysicalTensor, stream: Stream):
        return self._stamp(input, segment_offsets, stream, preallocated_index_output, True)


def segmented_broadcast(per_segment_values: PhysicalTensor, segment_offsets: PhysicalTensor, output: PhysicalTensor,
                        normalize_by_segment_length: bool, stream: Stream) -> None:
    """output[r] = per_segment_values[b] for the rows r of segment b = [offsets[b], offsets[b + 1]), divided by the segment's
    length when asked; rows of no segment keep their contents (reference: SegmentedBroadcastKernel.h launchSegmentedBroadcast)."""
    _check(lib().thor_segmented_broadcast(per_segment_values._h, segment_offsets._h, output._h, 1 if normalize_by_segment_length else 0, stream._h),
           "segmented_broadcast")


class RotaryScalingKind(enum.IntEnum):
    """thor.physical.RotaryScalingKind (Utilities/Expression/Expression.h:150-157 there)."""
    none = 0
    linear = 1
    dynamic_ntk = 2
    yarn = 3
    longrope = 4
    llama3 = 5


class _RopeOptions(ctypes.Structure):
    """thor_rope_options of the C-ABI."""
    _fields_ = [("sequence_axis", ctypes.c_uint32), ("head_dim_axis", ctypes.c_uint32), ("rotary_dim", ctypes.c_uint64), ("base", ctypes.c_double),
                ("position_offset", ctypes.c_int64), ("interleaved", ctypes.c_int), ("inverse", ctypes.c_int), ("scaling_kind", ctypes.c_int),
                ("scaling_factor", ctypes.c_double), ("original_max_position_embeddings", ctypes.c_uint64), ("attention_factor", ctypes.c_double),
                ("yarn_beta_fast", ctypes.c_double), ("yarn_beta_slow", ctypes.c_double), ("llama3_low_freq_factor", ctypes.c_double),
                ("llama3_high_freq_factor", ctypes.c_double), ("long_rope_short_factors", ctypes.POINTER(ctypes.c_double)),
                ("long_rope_long_factors", ctypes.POINTER(ctypes.c_double)), ("num_long_rope_factors", ctypes.c_uint64), ("output_dtype", ctypes.c_int),
                ("compute_dtype", ctypes.c_int)]


class ScanOp(enum.IntEnum):
    """thor.physical.ScanOp (Utilities/Expression/Expression.h:181-188 there)."""
    sum = 0
    min = 1
    max = 2
    product = 3
    arg_min = 4
    arg_max = 5


def scan(input: PhysicalTensor, output: PhysicalTensor, stream: Stream, op: ScanOp = ScanOp.sum, inclusive: bool = True, reverse: bool = False,
         segment_size: int = 0, segment_offsets: Optional[PhysicalTensor] = None, num_items: Optional[int] = None, no_alloc: bool = False) -> str:
    """Prefix scan of ``input`` into ``output``: flat, over rows of ``segment_size`` elements, or over the segments of an offsets
    tensor; ``ScanOp.arg_min`` / ``arg_max`` write UINT32 flattened indices (cubDeviceScan / cubDeviceSegmentedUniformScan /
    cubDeviceSegmentedScan and their arg forms, CubDevicePrimitives.h:781-880,951-1012 there).  Returns the kernel variant.
    ``no_alloc`` takes the entry point that allocates, compiles and loads nothing (temporary storage in the library's fixed
    scratch block; the kernels of the request must have been loaded by an ordinary scan before)."""
    n = int(num_items if num_items is not None else np.prod(input.get_dimensions()))
    arg = op in (ScanOp.arg_min, ScanOp.arg_max)
    code = {ScanOp.arg_min: 1, ScanOp.arg_max: 2}.get(op, int(op))
    segments = (segment_offsets.get_dimensions()[0] - 1) if segment_offsets is not None else (n // segment_size if segment_size else 1)
    text = ctypes.create_string_buffer(512)
    entry = lib().thor_scan_no_alloc if no_alloc else lib().thor_scan
    _check(entry(input._h, output._h, segment_offsets._h if segment_offsets is not None else None, n, segments, segment_size, code, int(arg),
                 int(inclusive), int(reverse), stream._h, text, 512), "scan")
    return text.value.decode()


def scan_waits_recovered() -> int:
    """How many bounded waits between the blocks of one-launch scans gave up, and recomputed what they waited for, over all
    ``scan`` calls of this process (a diagnostic; results are complete either way)."""
    return int(lib().thor_scan_waits_recovered())


class SelectionPlan:
    """A prepared select-flagged or top-k (prepareCubDeviceSelectFlagged / prepareCubDeviceTopKKeys / ...Pairs / Segmented..., the plan
    structs of CubDevicePrimitives.h:47-93 there): ``temp_storage_bytes`` of UINT8 temporary storage, ``run`` with the tensors in the
    order the plan was prepared with.  Nothing is allocated by ``run``."""

    def __init__(self, ptr, what):
        self._h = _handle(ptr, what)

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_selection_plan_destroy(self._h)
                self._h = None
        except Exception:
            pass

    @staticmethod
    def select_flagged(input: PhysicalTensor, flags: PhysicalTensor, output: PhysicalTensor, num_selected_out: PhysicalTensor,
                       num_items: Optional[int] = None) -> "SelectionPlan":
        n = int(num_items if num_items is not None else np.prod(input.get_dimensions()))
        return SelectionPlan(lib().thor_select_flagged_prepare(input._h, flags._h, output._h, num_selected_out._h, n), "prepare select_flagged")

    @staticmethod
    def top_k(keys_in: PhysicalTensor, keys_out: PhysicalTensor, k: int, largest: bool = True, values_in: Optional[PhysicalTensor] = None,
              values_out: Optional[PhysicalTensor] = None, num_items: Optional[int] = None, num_segments: Optional[int] = None,
              segment_size: Optional[int] = None) -> "SelectionPlan":
        values = (values_in._h if values_in is not None else None, values_out._h if values_out is not None else None)
        if segment_size is not None:
            segments = int(num_segments if num_segments is not None else np.prod(keys_in.get_dimensions()) // max(int(segment_size), 1))
            return SelectionPlan(lib().thor_topk_prepare(keys_in._h, keys_out._h, values[0], values[1], segments, int(segment_size), int(k), int(largest), 1),
                                 "prepare top_k")
        n = int(num_items if num_items is not None else np.prod(keys_in.get_dimensions()))
        return SelectionPlan(lib().thor_topk_prepare(keys_in._h, keys_out._h, values[0], values[1], 0, n, int(k), int(largest), 0), "prepare top_k")

    @property
    def temp_storage_bytes(self) -> int:
        return int(lib().thor_selection_plan_temp_bytes(self._h))

    def allocate_temp_storage(self, gpu_num: int = 0) -> PhysicalTensor:
        return PhysicalTensor(Placement(DeviceType.gpu, gpu_num), PhysicalTensor.Descriptor(DataType.uint8, [max(self.temp_storage_bytes, 1)]))

    def run(self, temp_storage: PhysicalTensor, a: PhysicalTensor, b: PhysicalTensor, c: Optional[PhysicalTensor] = None,
            d: Optional[PhysicalTensor] = None, *, stream: Stream):
        _check(lib().thor_selection_plan_run(self._h, temp_storage._h, a._h, b._h, c._h if c is not None else None, d._h if d is not None else None,
                                             stream._h), "SelectionPlan.run")

    def variant(self) -> str:
        text = ctypes.create_string_buffer(512)
        _check(lib().thor_selection_plan_variant(self._h, text, 512), "SelectionPlan.variant")
        return text.value.decode()


def select_flagged(input: PhysicalTensor, flags: PhysicalTensor, output: PhysicalTensor, num_selected_out: PhysicalTensor, stream: Stream,
                   num_items: Optional[int] = None) -> str:
    """``output`` receives the elements of ``input`` whose flag (BOOLEAN / UINT8) is nonzero, in input order, ``num_selected_out``
    (UINT32, one element) their number (cubDeviceSelectFlagged, CubDevicePrimitives.h:490-516 there).  Returns the kernel variant."""
    n = int(num_items if num_items is not None else np.prod(input.get_dimensions()))
    text = ctypes.create_string_buffer(512)
    _check(lib().thor_select_flagged(input._h, flags._h, output._h, num_selected_out._h, n, stream._h, text, 512), "select_flagged")
    return text.value.decode()


def top_k(keys_in: PhysicalTensor, keys_out: PhysicalTensor, k: int, stream: Stream, largest: bool = True,
          values_in: Optional[PhysicalTensor] = None, values_out: Optional[PhysicalTensor] = None, num_items: Optional[int] = None,
          num_segments: Optional[int] = None, segment_size: Optional[int] = None) -> str:
    """The ``k`` largest (or smallest) keys, unordered, with their UINT32 values when both value tensors are given
    (cubDeviceTopKKeys / cubDeviceTopKPairs, CubDevicePrimitives.h:357-420 there).  With ``segment_size`` the selection runs in
    every row of that many keys (at most 8192, ``k`` below it) and writes ``k`` keys per row (cubDeviceSegmentedTopKKeys / Pairs,
    :422-488 there).  Returns the kernel variant (empty when there is nothing to select)."""
    text = ctypes.create_string_buffer(512)
    values = (values_in._h if values_in is not None else None, values_out._h if values_out is not None else None)
    if segment_size is not None:
        segments = int(num_segments if num_segments is not None else np.prod(keys_in.get_dimensions()) // max(int(segment_size), 1))
        _check(lib().thor_topk(keys_in._h, keys_out._h, values[0], values[1], segments, int(segment_size), int(k), int(largest), 1, stream._h, text, 512),
               "top_k")
    else:
        n = int(num_items if num_items is not None else np.prod(keys_in.get_dimensions()))
        _check(lib().thor_topk(keys_in._h, keys_out._h, values[0], values[1], 0, n, int(k), int(largest), 0, stream._h, text, 512), "top_k")
    return text.value.decode()


# ---- expressions -------------------------------------------------------------------------------------------------------------
def _as_expr(value) -> "Expression":
    if isinstance(value, Expression):
        return value
    if isinstance(value, (int, float, np.floating, np.integer)):
        return Expression.constant_scalar(float(value))
    raise TypeError(f"cannot use {type(value).__name__} as an Expression operand")


def _parse_axes(axis) -> List[int]:
    if axis is None:
        return []
    if isinstance(axis, (int, np.integer)):
        return [int(axis)]
    return [int(a) for a in axis]


def _parse_squeeze(squeeze) -> List[int]:
    if squeeze is True:
        return [UINT64_MAX]
    if squeeze is False or squeeze is None:
        return []
    if isinstance(squeeze, (int, np.integer)):
        return [int(squeeze)]
    return [int(a) for a in squeeze]


class Expression:
    """Expression graph node; static builders mirror `thor.physical.Expression` (`ex.input`, `ex.exp`, `ex.reduce_sum`, ...)."""

    def __init__(self, ptr):
        self._h = _handle(ptr, "Expression")

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_expr_destroy(self._h)
                self._h = None
        except Exception:
            pass

    # -- leaves
    @staticmethod
    def input(name: str, compute_dtype: Optional[DataType] = None, output_dtype: Optional[DataType] = None) -> "Expression":
        return Expression(lib().thor_expr_input(name.encode(), _dtype_code(compute_dtype), _dtype_code(output_dtype)))

    @staticmethod
    def runtime_scalar(name: str, compute_dtype: Optional[DataType] = None, output_dtype: Optional[DataType] = None) -> "Expression":
        return Expression(lib().thor_expr_runtime_scalar(name.encode(), _dtype_code(compute_dtype), _dtype_code(output_dtype)))

    @staticmethod
    def tensor_runtime_scalar(name: str, compute_dtype: Optional[DataType] = None, output_dtype: Optional[DataType] = None) -> "Expression":
        """A scalar read from device memory at every run; bound at stamp time with a TensorScalarBinding."""
        return Expression(_handle(lib().thor_expr_tensor_runtime_scalar(name.encode(), _dtype_code(compute_dtype), _dtype_code(output_dtype)),
                                  "tensor_runtime_scalar"))

    @staticmethod
    def constant_scalar(value: float) -> "Expression":
        return Expression(lib().thor_expr_scalar(float(value)))

    @staticmethod
    def fill(value: float, dims: Sequence[int], output_dtype: Optional[DataType] = None) -> "Expression":
        d, rank = _u64_array(dims)
        return Expression(lib().thor_expr_fill(float(value), d, rank, _dtype_code(output_dtype)))

    # -- generic dispatch
    def _binary(self, method: str, other, reflected: bool = False) -> "Expression":
        other = _as_expr(other)
        lhs, rhs = (other, self) if reflected else (self, other)
        return Expression(lib().thor_expr_binary(method.encode(), lhs._h, rhs._h))

    def _unary(self, method: str) -> "Expression":
        return Expression(lib().thor_expr_unary(method.encode(), self._h))

    def __add__(self, o): return self._binary("add", o)
    def __radd__(self, o): return self._binary("add", o, True)
    def __sub__(self, o): return self._binary("sub", o)
    def __rsub__(self, o): return self._binary("sub", o, True)
    def __mul__(self, o): return self._binary("mul", o)
    def __rmul__(self, o): return self._binary("mul", o, True)
    def __truediv__(self, o): return self._binary("div", o)
    def __rtruediv__(self, o): return self._binary("div", o, True)
    def __pow__(self, o): return self._binary("pow", o)
    def __rpow__(self, o): return self._binary("pow", o, True)
    def __neg__(self): return self._unary("neg")
    def __lt__(self, o): return self._binary("lessThan", o)
    def __le__(self, o): return self._binary("lessEqual", o)
    def __gt__(self, o): return self._binary("greaterThan", o)
    def __ge__(self, o): return self._binary("greaterEqual", o)
    def __eq__(self, o): return self._binary("equal", o)  # type: ignore[override]
    def __ne__(self, o): return self._binary("notEqual", o)  # type: ignore[override]
    __hash__ = None  # type: ignore[assignment]

    def min(self, o): return self._binary("min", o)
    def max(self, o): return self._binary("max", o)
    def pow(self, o): return self._binary("pow", o)
    def logical_and(self, o): return self._binary("logicalAnd", o)
    def logical_or(self, o): return self._binary("logicalOr", o)
    def logical_not(self): return self._unary("logicalNot")
    def dot_product(self, o): return self._binary("dotProduct", o)

    def cast(self, dtype: DataType) -> "Expression":
        return Expression(lib().thor_expr_cast(self._h, int(dtype)))

    def with_dtypes(self, compute_dtype: Optional[DataType] = None, output_dtype: Optional[DataType] = None) -> "Expression":
        return Expression(lib().thor_expr_with_dtypes(self._h, _dtype_code(compute_dtype), _dtype_code(output_dtype)))

    def with_compute_dtype(self, dtype: DataType) -> "Expression":
        return self.with_dtypes(compute_dtype=dtype)

    def with_output_dtype(self, dtype: DataType) -> "Expression":
        return self.with_dtypes(output_dtype=dtype)

    @staticmethod
    def where(condition, true_value, false_value) -> "Expression":
        return Expression(lib().thor_expr_where(_as_expr(condition)._h, _as_expr(true_value)._h, _as_expr(false_value)._h))

    select = where

    def elu(self, alpha: float = 1.0): return Expression(lib().thor_expr_unary_params(b"elu", self._h, alpha, 0.0))
    def hard_tanh(self, min_value=-1.0, max_value=1.0): return Expression(lib().thor_expr_unary_params(b"hardTanh", self._h, min_value, max_value))
    def threshold(self, threshold=0.0, value=0.0): return Expression(lib().thor_expr_unary_params(b"threshold", self._h, threshold, value))
    def log(self, base: float): return Expression(lib().thor_expr_unary_params(b"log", self._h, base, 0.0))
    def clamp(self, lo: float, hi: float): return Expression(lib().thor_expr_unary_params(b"clamp", self._h, lo, hi))

    def softmax(self, algorithm: str = "accurate", mode: str = "channel") -> "Expression":
        """Softmax over axis 1 ("channel") or over every axis but the first ("instance"); "fast" skips the max subtraction."""
        return Expression(lib().thor_expr_unary_params(b"softmax", self._h, {"fast": 0.0, "accurate": 1.0}[algorithm], {"instance": 0.0, "channel": 1.0}[mode]))

    def log_softmax(self, mode: str = "channel") -> "Expression":
        return Expression(lib().thor_expr_unary_params(b"logSoftmax", self._h, 1.0, {"instance": 0.0, "channel": 1.0}[mode]))

    # -- ragged batches: values [N, D...] packed row after row, offsets [B + 1] read on the device when the plan runs
    def _ragged(self, method: str, offsets: "Expression", batch_size: int, max_active_values: int, elements_per_value: int) -> "Expression":
        return Expression(lib().thor_expr_ragged(method.encode(), self._h, offsets._h, batch_size, max_active_values, elements_per_value))

    def segment_sum(self, offsets, batch_size=0, max_active_values=0, elements_per_value=1):
        """Per-segment sum -> [B, D...] in the values' dtype (fp32 accumulation); empty segments give 0."""
        return self._ragged("segment_sum", offsets, batch_size, max_active_values, elements_per_value)

    def segment_min(self, offsets, batch_size=0, max_active_values=0, elements_per_value=1):
        return self._ragged("segment_min", offsets, batch_size, max_active_values, elements_per_value)

    def segment_max(self, offsets, batch_size=0, max_active_values=0, elements_per_value=1):
        return self._ragged("segment_max", offsets, batch_size, max_active_values, elements_per_value)

    def segment_mean(self, offsets, batch_size=0, max_active_values=0, elements_per_value=1):
        return self._ragged("segment_mean", offsets, batch_size, max_active_values, elements_per_value)

    def segmented_broadcast(self, offsets, batch_size: int, max_active_values: int, elements_per_value: int = 1, normalize_by_segment_length: bool = False):
        """Per-segment values [B, D...] -> rows [max_active_values, D...]; rows of no segment are undefined."""
        method = "segmented_broadcast_normalized" if normalize_by_segment_length else "segmented_broadcast"
        return self._ragged(method, offsets, batch_size, max_active_values, elements_per_value)

    def with_ragged_runtime_extent(self, offsets, batch_size: int, max_active_values: int, elements_per_value: int = 1):
        """The same values, computed only for the first offsets[batch_size] rows; the rest of the output keeps its contents."""
        return self._ragged("ragged_extent", offsets, batch_size, max_active_values, elements_per_value)

    def scan(self, op: "ScanOp" = None, axis: int = -1, inclusive: bool = True, reverse: bool = False) -> "Expression":
        """Prefix scan along the last axis; values keep their dtype, ``ScanOp.arg_min`` / ``arg_max`` return UINT32 flattened
        indices (thor.physical.Expression.scan)."""
        op = ScanOp.sum if op is None else op
        return Expression(_handle(lib().thor_expr_scan(self._h, None, int(op), axis, int(inclusive), int(reverse)), "scan"))

    def segmented_scan(self, offsets: "Expression", op: "ScanOp" = None, inclusive: bool = True, reverse: bool = False) -> "Expression":
        op = ScanOp.sum if op is None else op
        return Expression(_handle(lib().thor_expr_scan(self._h, offsets._h, int(op), -1, int(inclusive), int(reverse)), "segmented_scan"))

    def scan_with_indices(self, op: "ScanOp", axis: int = -1, inclusive: bool = True):
        if op not in (ScanOp.min, ScanOp.max):
            raise ValueError("scan_with_indices supports only ScanOp.min and ScanOp.max")
        return self.scan(op, axis, inclusive), self.scan(ScanOp.arg_min if op == ScanOp.min else ScanOp.arg_max, axis, inclusive)

    def segmented_scan_with_indices(self, offsets: "Expression", op: "ScanOp", inclusive: bool = True, reverse: bool = False):
        if op not in (ScanOp.min, ScanOp.max):
            raise ValueError("segmented_scan_with_indices supports only ScanOp.min and ScanOp.max")
        return (self.segmented_scan(offsets, op, inclusive, reverse),
                self.segmented_scan(offsets, ScanOp.arg_min if op == ScanOp.min else ScanOp.arg_max, inclusive, reverse))

    def prefix_count(self, inclusive: bool = True, axis: int = -1) -> "Expression":
        return self.cast(DataType.uint32).scan(ScanOp.sum, axis, inclusive)

    def take_along_axis(self, indices: "Expression", axis: int = -1) -> "Expression":
        """Gather along one axis with UINT32 / UINT64 indices; the result has the shape of ``indices``."""
        return Expression(_handle(lib().thor_expr_take_along_axis(self._h, indices._h, axis), "take_along_axis"))

    def rope(self, sequence_axis: int = 2, head_dim_axis: int = 3, rotary_dim: int = 0, base: float = 10000.0, position_offset: int = 0,
             interleaved: bool = False, inverse: bool = False, scaling_kind: "RotaryScalingKind" = None, scaling_factor: float = 1.0,
             original_max_position_embeddings: int = 0, attention_factor: Optional[float] = None, yarn_beta_fast: float = 32.0,
             yarn_beta_slow: float = 1.0, llama3_low_freq_factor: float = 1.0, llama3_high_freq_factor: float = 4.0,
             long_rope_short_factors: Sequence[float] = (), long_rope_long_factors: Sequence[float] = (), output_dtype: Optional[DataType] = None,
             compute_dtype: Optional[DataType] = None, allow_in_place_materialization: bool = False, position_ids: Optional["Expression"] = None,
             effective_sequence_length: Optional["Expression"] = None) -> "Expression":
        """Rotary position embedding (thor.physical.Expression.rope / rotary_position_embedding: bindings/python/src/core/physical/
        expression.cpp:1233-1385 there).  ``rotary_dim=0`` turns the whole head dimension.  ``position_ids`` (one absolute position
        per element of the sequence axis) and ``effective_sequence_length`` (one element) are the C++ API's WithPositionIds /
        WithEffectiveSequenceLength forms."""
        if attention_factor is not None and attention_factor <= 0:
            raise RuntimeError("RoPE attention_factor must be positive.")
        if len(long_rope_short_factors) != len(long_rope_long_factors):
            raise RuntimeError("LongRoPE scaling requires short/long factor lists of length rotary_dim / 2.")
        count = len(long_rope_short_factors)
        short = (ctypes.c_double * max(count, 1))(*[float(v) for v in long_rope_short_factors])
        long_ = (ctypes.c_double * max(count, 1))(*[float(v) for v in long_rope_long_factors])
        options = _RopeOptions(int(sequence_axis), int(head_dim_axis), int(rotary_dim), float(base), int(position_offset), int(bool(interleaved)),
                               int(bool(inverse)), int(RotaryScalingKind.none if scaling_kind is None else scaling_kind), float(scaling_factor),
                               int(original_max_position_embeddings), float(attention_factor) if attention_factor is not None else 0.0,
                               float(yarn_beta_fast), float(yarn_beta_slow), float(llama3_low_freq_factor), float(llama3_high_freq_factor),
                               ctypes.cast(short, ctypes.POINTER(ctypes.c_double)), ctypes.cast(long_, ctypes.POINTER(ctypes.c_double)), count,
                               -1 if output_dtype is None else int(output_dtype), -1 if compute_dtype is None else int(compute_dtype))
        ids = position_ids._h if position_ids is not None else None
        length = effective_sequence_length._h if effective_sequence_length is not None else None
        return Expression(_handle(lib().thor_expr_rope(self._h, ids, length, ctypes.byref(options)), "rope"))

    rotary_position_embedding = rope

    def transpose(self) -> "Expression":
        """The last two axes exchanged, as a view of the operand's storage."""
        return self._unary("transpose")

    def strided_view(self, dims: Sequence[int], strides_elements: Sequence[int], element_offset: int = 0) -> "Expression":
        """A view of the operand's storage: strides and offset are in elements of the tensor the operand resolves to."""
        d, rank = _u64_array(dims)
        st, rank2 = _u64_array(strides_elements)
        if rank != rank2:
            raise ValueError("strided_view needs one stride per dimension")
        return Expression(lib().thor_expr_strided_view(self._h, d, st, rank, int(element_offset)))

    alias_view = strided_view

    def reshape(self, dims: Sequence[int]) -> "Expression":
        d, rank = _u64_array([UINT64_MAX if v == -1 else v for v in dims])
        return Expression(lib().thor_expr_reshape(self._h, d, rank))

    def unsqueeze(self, axes) -> "Expression":
        a, n = _u64_array(_parse_axes(axes))
        return Expression(lib().thor_expr_unsqueeze(self._h, a, n))

    def squeeze(self, axes) -> "Expression":
        a, n = _u64_array(_parse_axes(axes))
        return Expression(lib().thor_expr_squeeze(self._h, a, n))

    def _reduce(self, method: str, axis=None, squeeze=False, output_dtype: Optional[DataType] = None) -> "Expression":
        axes, na = _u64_array(_parse_axes(axis))
        sq, ns = _u64_array(_parse_squeeze(squeeze))
        out = Expression(lib().thor_expr_reduce(method.encode(), self._h, axes, na, sq, ns))
        return out.with_output_dtype(output_dtype) if output_dtype is not None else out

    def num_nodes(self) -> int:
        return lib().thor_expr_num_nodes(self._h)

    def canonical(self) -> str:
        need = ctypes.c_size_t()
        cap = 1 << 16
        buf = ctypes.create_string_buffer(cap)
        _check(lib().thor_expr_canonical(self._h, buf, cap, ctypes.byref(need)), "canonical")
        return buf.value.decode()

    # -- compile (thor.physical.Expression.compile)
    @staticmethod
    def outputs(named: Dict[str, "Expression"]) -> "Outputs":
        return Outputs(named)

    @staticmethod
    def if_else(predicate: "Expression", then_outputs: "Outputs", else_outputs: "Outputs") -> "Outputs":
        """Outputs that take the then-branch's values where the single-element ``predicate`` is nonzero at run time, the
        else-branch's otherwise (thor.physical.Expression.if_else; both branches are evaluated here and selected element by element)."""
        return Outputs._conditional(predicate, then_outputs, [], else_outputs)

    conditional = if_else

    @staticmethod
    def if_elif_else(predicate: "Expression", then_outputs: "Outputs", elif_branches, else_outputs: "Outputs") -> "Outputs":
        if not elif_branches:
            raise RuntimeError("Outputs::ifElifElse requires at least one elif branch.")
        return Outputs._conditional(predicate, then_outputs, list(elif_branches), else_outputs)

    @staticmethod
    def compile(expr_or_outputs, device_num: int = 0) -> "FusedEquation":
        outputs = expr_or_outputs if isinstance(expr_or_outputs, Outputs) else Outputs({"output": _as_expr(expr_or_outputs)})
        return FusedEquation(_handle(lib().thor_fused_equation_compile(outputs._h, device_num), "Expression.compile"))


_UNARY_NAMES = ["abs", "ceil", "floor", "round", "trunc", "sin", "cos", "tan", "csc", "sec", "cot", "asin", "acos", "atan", "acsc", "asec", "acot",
                "sinh", "cosh", "tanh", "csch", "sech", "coth", "asinh", "acosh", "atanh", "acsch", "asech", "acoth", "erf", "erfc", "erfcx",
                "erfinv", "erfcinv", "tgamma", "lgamma", "digamma", "ln", "log1p", "log2", "log10", "exp", "expm1", "exp2", "exp10", "sqrt",
                "normcdf", "sigmoid", "softplus", "selu", "gelu", "mish", "relu6", "swish"]
for _name in _UNARY_NAMES:
    setattr(Expression, _name, (lambda n: lambda self: self._unary(n))(_name))
Expression.hard_swish = lambda self: self._unary("hardSwish")
Expression.relu = lambda self: self.max(0.0)  # ReLU is spelled max(x, 0) in the reference (Api/Layers/Activations/Relu.h:21-22)

_REDUCTIONS = ["reduce_sum", "reduce_prod", "reduce_min", "reduce_max", "reduce_mean", "reduce_norm1", "reduce_norm2"]
for _name in _REDUCTIONS:
    setattr(Expression, _name, (lambda n: lambda self, axis=None, squeeze=False, compute_dtype=DataType.fp32, output_dtype=DataType.fp32:
                                self._reduce(n, axis, squeeze, output_dtype))(_name))
Expression.argmin = lambda self, axis=None, squeeze=False: self._reduce("argmin", axis, squeeze)
Expression.argmax = lambda self, axis=None, squeeze=False: self._reduce("argmax", axis, squeeze)


class Outputs:
    def __init__(self, named: Dict[str, Expression]):
        names = list(named.keys())
        self._h = _handle(lib().thor_outputs_create(_names(names), _ptrs([named[n]._h for n in names]), len(names)), "Expression.outputs")

    @staticmethod
    def _conditional(predicate: Expression, then_outputs: "Outputs", elif_branches, else_outputs: "Outputs") -> "Outputs":
        out = Outputs.__new__(Outputs)
        out._h = _handle(lib().thor_outputs_conditional(_as_expr(predicate)._h, then_outputs._h, _ptrs([_as_expr(p)._h for p, _ in elif_branches]),
                                                        _ptrs([o._h for _, o in elif_branches]), len(elif_branches), else_outputs._h), "Outputs.conditional")
        return out

    def compile(self, device_num: int = 0) -> "FusedEquation":
        return Expression.compile(self, device_num)

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_outputs_destroy(self._h)
                self._h = None
        except Exception:
            pass


class Equation:
    """A stamped execution plan (StampedExecutionPlan): run() only launches."""

    def __init__(self, ptr):
        self._h = ptr

    def run(self, runtime_scalars: Optional[Dict[str, float]] = None):
        if runtime_scalars:
            names = list(runtime_scalars)
            vals = (ctypes.c_float * len(names))(*[runtime_scalars[n] for n in names])
            _check(lib().thor_plan_run_with_scalars(self._h, _names(names), vals, len(names)), "Equation.run")
        else:
            _check(lib().thor_plan_run(self._h), "Equation.run")

    def run_on(self, stream: Stream):
        _check(lib().thor_plan_run_on(self._h, stream._h), "Equation.runOn")

    def output(self, name: Optional[str] = None) -> PhysicalTensor:
        return PhysicalTensor._wrap(lib().thor_plan_output(self._h, name.encode() if name is not None else None))

    def stage_kind_names(self) -> List[str]:
        out = []
        for s in range(lib().thor_plan_num_stages(self._h)):
            buf = ctypes.create_string_buffer(64)
            _check(lib().thor_plan_stage_kind(self._h, s, buf, 64), "stageKindNames")
            out.append(buf.value.decode())
        return out

    def stage_descriptions(self) -> List[str]:
        out = []
        for s in range(lib().thor_plan_num_stages(self._h)):
            buf = ctypes.create_string_buffer(512)
            _check(lib().thor_plan_stage_description(self._h, s, buf, 512), "stage description")
            out.append(buf.value.decode())
        return out

    def stage_source(self, stage: int) -> str:
        cap = 1 << 20
        buf = ctypes.create_string_buffer(cap)
        need = ctypes.c_size_t()
        _check(lib().thor_plan_stage_source(self._h, stage, buf, cap, ctypes.byref(need)), "stage source")
        return buf.value.decode()

    def flop_count(self) -> int:
        return lib().thor_plan_flop_count(self._h)

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_plan_destroy(self._h)
                self._h = None
        except Exception:
            pass


class TensorScalarBinding:
    """thor.physical.TensorScalarBinding: one element of ``source_dtype`` at ``byte_offset`` inside ``buffer``."""

    def __init__(self, buffer: Optional[PhysicalTensor] = None, byte_offset: int = 0, source_dtype: DataType = DataType.fp32):
        self.buffer = buffer
        self.byte_offset = byte_offset
        self.source_dtype = source_dtype


class FusedEquation:
    def __init__(self, ptr):
        self._h = ptr

    def output_names(self) -> List[str]:
        out = []
        for i in range(lib().thor_fused_equation_num_outputs(self._h)):
            buf = ctypes.create_string_buffer(256)
            _check(lib().thor_fused_equation_output_name(self._h, i, buf, 256), "getOutputNames")
            out.append(buf.value.decode())
        return out

    def compile_backward(self, wrt_names: Optional[List[str]] = None,
                         error_input_name: Union[None, str, Dict[str, str]] = None, accumulate_grad_outputs: bool = False) -> "FusedEquation":
        """Equation of the gradients ``<input>_grad`` of ``wrt_names`` (all tensor inputs when empty).

        ``error_input_name`` names the upstream gradient input of a single-output equation, or maps forward output names to
        upstream gradient input names; None means implicit ones for a single output.  (reference:
        bindings/python/src/core/physical/expression.cpp:2638-2720)
        """
        wrt = list(wrt_names or [])
        if isinstance(error_input_name, dict):
            if len(error_input_name) == 0:
                raise RuntimeError("Cannot compute backward expression with no error inputs.")
            outs = list(error_input_name)
            ptr = lib().thor_fused_equation_compile_backward(self._h, _names(wrt), len(wrt), _names(outs), _names([error_input_name[o] for o in outs]),
                                                             len(outs), int(accumulate_grad_outputs))
        elif error_input_name is None:
            ptr = lib().thor_fused_equation_compile_backward(self._h, _names(wrt), len(wrt), None, None, 0, int(accumulate_grad_outputs))
        else:
            ptr = lib().thor_fused_equation_compile_backward(self._h, _names(wrt), len(wrt), None, _names([error_input_name]), 1,
                                                             int(accumulate_grad_outputs))
        return FusedEquation(_handle(ptr, "FusedEquation.compile_backward"))

    def stamp(self, inputs: Dict[str, PhysicalTensor], stream: Stream, preallocated_outputs: Optional[Dict[str, PhysicalTensor]] = None,
              tensor_scalar_inputs: Optional[Dict[str, TensorScalarBinding]] = None) -> Equation:
        names = list(inputs)
        pre = preallocated_outputs or {}
        pre_names = list(pre)
        if tensor_scalar_inputs:
            s_names = list(tensor_scalar_inputs)
            bindings = [tensor_scalar_inputs[n] for n in s_names]
            offsets = (ctypes.c_uint64 * len(s_names))(*[int(b.byte_offset) for b in bindings])
            dtypes = (ctypes.c_int * len(s_names))(*[int(b.source_dtype) for b in bindings])
            ptr = lib().thor_fused_equation_stamp_with_tensor_scalars(
                self._h, _names(names), _ptrs([inputs[n]._h for n in names]), len(names), _names(s_names), _ptrs([b.buffer._h for b in bindings]), offsets,
                dtypes, len(s_names), _names(pre_names), _ptrs([pre[n]._h for n in pre_names]), len(pre_names), stream._h)
            return Equation(_handle(ptr, "FusedEquation.stamp"))
        ptr = lib().thor_fused_equation_stamp(self._h, _names(names), _ptrs([inputs[n]._h for n in names]), len(names), _names(pre_names),
                                              _ptrs([pre[n]._h for n in pre_names]), len(pre_names), stream._h)
        return Equation(_handle(ptr, "FusedEquation.stamp"))

    def run(self, inputs: Union[PhysicalTensor, Dict[str, PhysicalTensor]], outputs: Union[PhysicalTensor, Dict[str, PhysicalTensor]], stream: Stream,
            scalar_inputs: Optional[Dict[str, float]] = None):
        if isinstance(outputs, PhysicalTensor):
            out_names = self.output_names()
            if len(out_names) != 1:
                raise RuntimeError("run(..., output) requires an equation with exactly one output")
            outputs = {out_names[0]: outputs}
        if isinstance(inputs, PhysicalTensor):
            raise TypeError("pass inputs as a {name: tensor} dict")
        in_names, out_names = list(inputs), list(outputs)
        scalars = scalar_inputs or {}
        s_names = list(scalars)
        s_vals = (ctypes.c_float * max(1, len(s_names)))(*[scalars[n] for n in s_names])
        _check(lib().thor_fused_equation_run(self._h, _names(in_names), _ptrs([inputs[n]._h for n in in_names]), len(in_names), _names(s_names), s_vals,
                                             len(s_names), _names(out_names), _ptrs([outputs[n]._h for n in out_names]), len(out_names), stream._h),
               "FusedEquation.run")

    def get_output_shape(self, inputs: Dict[str, PhysicalTensor], output_name: str = "output"):
        names = list(inputs)
        dims = (ctypes.c_uint64 * 16)()
        rank, dtype = ctypes.c_int(), ctypes.c_int()
        _check(lib().thor_fused_equation_output_shape(self._h, _names(names), _ptrs([inputs[n]._h for n in names]), len(names), output_name.encode(), dims,
                                                      ctypes.byref(rank), ctypes.byref(dtype)), "getOutputShape")
        return list(dims[: rank.value]), DataType(dtype.value)

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                lib().thor_fused_equation_destroy(self._h)
                self._h = None
        except Exception:
            pass


def compiled_kernel_count() -> int:
    return lib().thor_compiled_kernel_count()
