"""Shared helpers of the GPU parity tests; shaped after the reference's python test helpers
(bindings/python/test/core/physical/test_expression_numerical.py:40-120)."""
from __future__ import annotations

import numpy as np

import oracle
from thor_amd import physical as ph
from thor_amd.dtypes import DataType, numpy_carrier

FLOAT_DTYPES = [DataType.fp16, DataType.bf16, DataType.fp8_e4m3, DataType.fp8_e5m2, DataType.fp32]


def cpu_tensor(shape, dtype):
    return ph.PhysicalTensor(ph.Placement(ph.DeviceType.cpu, 0), ph.PhysicalTensor.Descriptor(dtype, list(shape)))


def gpu_tensor(shape, dtype, gpu_num=0):
    return ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, gpu_num), ph.PhysicalTensor.Descriptor(dtype, list(shape)))


def to_storage(values_f32: np.ndarray, dtype: DataType) -> np.ndarray:
    """fp32 values -> carrier array of `dtype` (RNE through the oracle's converters)."""
    values_f32 = np.ascontiguousarray(values_f32, dtype=np.float32)
    if dtype == DataType.fp32:
        return values_f32
    return oracle.convert(values_f32, oracle.FP32, int(dtype)).reshape(values_f32.shape)


def from_storage(carrier: np.ndarray, dtype: DataType) -> np.ndarray:
    """carrier array -> fp32 (or the native integer values)."""
    if dtype in (DataType.fp16, DataType.bf16, DataType.fp8_e4m3, DataType.fp8_e5m2):
        return oracle.convert(np.ascontiguousarray(carrier), int(dtype), oracle.FP32).reshape(carrier.shape)
    return carrier


def copy_numpy_to_gpu(carrier: np.ndarray, stream, dtype: DataType, gpu_num=0):
    carrier = np.ascontiguousarray(carrier, dtype=numpy_carrier(dtype))
    shape = list(carrier.shape) if carrier.ndim else [1]
    cpu = cpu_tensor(shape, dtype)
    cpu.numpy()[...] = carrier.reshape(shape)
    gpu = gpu_tensor(shape, dtype, gpu_num)
    gpu.copy_from_async(cpu, stream)
    stream.synchronize()
    return gpu


def copy_gpu_to_numpy(t, stream) -> np.ndarray:
    dtype = t.get_data_type()
    if not t.is_dense_contiguous():
        raise AssertionError("download helper needs a dense tensor")
    cpu = cpu_tensor(t.get_dimensions(), dtype)
    cpu.copy_from_async(t, stream)
    stream.synchronize()
    return np.array(cpu.numpy(), copy=True)


def f32_to_gpu(values: np.ndarray, dtype: DataType, stream):
    return copy_numpy_to_gpu(to_storage(values, dtype), stream, dtype)


def gpu_to_f32(t, stream) -> np.ndarray:
    return from_storage(copy_gpu_to_numpy(t, stream), t.get_data_type())


def rtol_atol(dtype: DataType):
    """Per-dtype tolerances of the reference's numerical tests (test_expression_numerical.py:24-38)."""
    return {DataType.fp32: (3e-5, 3e-6), DataType.fp16: (5e-3, 5e-3), DataType.bf16: (2e-2, 2e-2), DataType.fp8_e4m3: (1.5e-1, 1.5e-1),
            DataType.fp8_e5m2: (2.5e-1, 2.5e-1)}[dtype]


def ulp_distance_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Distance in units in the last place between fp32 arrays (NaN == NaN, signed zeros equal)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)

    def ordered(x):
        i = x.view(np.int32).astype(np.int64)
        return np.where(i < 0, -(i & 0x7FFFFFFF), i)
    d = np.abs(ordered(a) - ordered(b))
    both_nan = np.isnan(a) & np.isnan(b)
    return np.where(both_nan, 0, d)


def run_expr(expr, inputs: dict, dtype: DataType, out_shape=None, out_dtype=None, scalars=None):
    """compile + FusedEquation.run into a caller-provided output (the reference's `_run_expr`)."""
    stream = ph.Stream(0)
    eq = ph.Expression.compile(expr, device_num=0)
    gpu_inputs = {k: copy_numpy_to_gpu(v, stream, dtype if not isinstance(dtype, dict) else dtype[k]) for k, v in inputs.items()}
    first = next(iter(inputs.values()))
    out = gpu_tensor(list(out_shape if out_shape is not None else first.shape), out_dtype or (dtype if not isinstance(dtype, dict) else None))
    eq.run(gpu_inputs, out, stream, scalar_inputs=scalars)
    return copy_gpu_to_numpy(out, stream)


def run_staged(expr_or_outputs, inputs: dict, dtypes, preallocated=None, scalars=None):
    """compile + stamp + run (the reference's `_run_staged_expr`); returns (plan, {name: carrier array})."""
    stream = ph.Stream(0)
    eq = ph.Expression.compile(expr_or_outputs, device_num=0)
    gpu_inputs = {k: copy_numpy_to_gpu(v, stream, dtypes[k] if isinstance(dtypes, dict) else dtypes) for k, v in inputs.items()}
    plan = eq.stamp(gpu_inputs, stream, preallocated_outputs=preallocated)
    plan.run(scalars)
    outs = {name: copy_gpu_to_numpy(plan.output(name), stream) for name in eq.output_names()}
    return plan, outs
