"""Expression.tensor_runtime_scalar: scalars that live in device memory and are read at every run
(bindings/python/test/core/physical/test_expression_tensor_scalar_inputs.py:80-200 there)."""
from __future__ import annotations

import numpy as np
import pytest

from helpers import FLOAT_DTYPES, copy_gpu_to_numpy, copy_numpy_to_gpu, cpu_tensor, from_storage, gpu_tensor, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex, TensorScalarBinding

pytestmark = pytest.mark.gpu
TOLERANCE = {DataType.fp32: (1e-5, 1e-6), DataType.fp16: (5e-3, 5e-3), DataType.bf16: (5e-3, 5e-3), DataType.fp8_e4m3: (1e-1, 1e-1),
             DataType.fp8_e5m2: (1e-1, 1e-1)}


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def overwrite(tensor, values, dtype, stream):
    host = cpu_tensor(list(values.shape), dtype)
    host.numpy()[...] = values
    tensor.copy_from_async(host, stream)
    stream.synchronize()


@pytest.mark.parametrize("dtype", FLOAT_DTYPES, ids=lambda d: d.name)
def test_stamped_plan_reads_the_buffer_at_its_byte_offset_on_every_run(stream, dtype):
    x = to_storage(np.array([[1.0, 2.0, 3.0], [4.0, -5.0, 6.5]], np.float32), dtype)
    xf = from_storage(x, dtype)
    out = ex.input("x") * ex.tensor_runtime_scalar("step") + ex.constant_scalar(1.0)
    buffer = copy_numpy_to_gpu(np.array([123.0, 0.25], np.float32), stream, DataType.fp32)
    plan = ex.compile(out, device_num=0).stamp({"x": copy_numpy_to_gpu(x, stream, dtype)}, stream,
                                               tensor_scalar_inputs={"step": TensorScalarBinding(buffer, byte_offset=4, source_dtype=DataType.fp32)})
    assert plan.stage_kind_names() == ["FusedKernel"] and "flat" in plan.stage_descriptions()[0]  # the scalar does not break the flat kernel
    assert plan.output().get_data_type() == dtype  # a scalar takes no part in dtype promotion
    rtol, atol = TOLERANCE[dtype]
    plan.run()
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(plan.output(), stream), dtype), from_storage(to_storage(xf * 0.25 + 1.0, dtype), dtype), rtol=rtol, atol=atol)
    overwrite(buffer, np.array([123.0, -1.5], np.float32), DataType.fp32, stream)  # other GPU work updates the value: the same plan follows it
    plan.run()
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(plan.output(), stream), dtype), from_storage(to_storage(xf * -1.5 + 1.0, dtype), dtype), rtol=rtol, atol=atol)


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16], ids=lambda d: d.name)
def test_several_outputs_preallocated_and_a_large_flat_kernel(stream, dtype):
    rng = np.random.default_rng(61)
    x = to_storage(rng.standard_normal((1000, 777)).astype(np.float32), dtype)
    xf = from_storage(x, dtype).astype(np.float64)
    ix, step = ex.input("x"), ex.tensor_runtime_scalar("step")
    outputs = ex.outputs({"scaled": ix * step, "shifted": ix + step, "row_sums": (ix * step).reduce_sum(axis=1)})
    pre = {"scaled": gpu_tensor([1000, 777], dtype), "shifted": gpu_tensor([1000, 777], dtype)}
    buffer = copy_numpy_to_gpu(np.array([-1.5], np.float32), stream, DataType.fp32)
    plan = ex.compile(outputs, device_num=0).stamp({"x": copy_numpy_to_gpu(x, stream, dtype)}, stream, preallocated_outputs=pre,
                                                   tensor_scalar_inputs={"step": TensorScalarBinding(buffer, 0, DataType.fp32)})
    plan.run()
    tolerance = 1e-6 if dtype == DataType.fp32 else 2e-3
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(pre["scaled"], stream), dtype), xf * -1.5, rtol=tolerance, atol=tolerance)
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(pre["shifted"], stream), dtype), xf - 1.5, rtol=tolerance, atol=tolerance)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("row_sums"), stream).reshape(-1), (xf * -1.5).sum(axis=1), rtol=2e-3, atol=2e-2 if dtype == DataType.fp32 else 0.1)  # fp16 products round before they are summed


def test_scalars_of_other_dtypes_and_backward(stream):
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    scale16 = copy_numpy_to_gpu(to_storage(np.array([0.5, 3.0], np.float32), DataType.fp16), stream, DataType.fp16)
    forward = ex.compile((ex.input("x") * ex.tensor_runtime_scalar("scale")).exp(), device_num=0)
    binding = {"scale": TensorScalarBinding(scale16, 0, DataType.fp16)}
    plan = forward.stamp({"x": copy_numpy_to_gpu(x, stream, DataType.fp32)}, stream, tensor_scalar_inputs=binding)
    plan.run()
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output(), stream), np.exp(x * 0.5), rtol=2e-6)
    backward = forward.compile_backward(["x"]).stamp({"x": copy_numpy_to_gpu(x, stream, DataType.fp32)}, stream, tensor_scalar_inputs=binding)
    backward.run()
    np.testing.assert_allclose(copy_gpu_to_numpy(backward.output("x_grad"), stream), 0.5 * np.exp(x * 0.5), rtol=2e-6)
    with pytest.raises(RuntimeError, match="only supports gradients with respect to tensor inputs"):
        forward.compile_backward(["scale"])


def test_binding_validation(stream):
    x = copy_numpy_to_gpu(np.ones((2, 2), np.float32), stream, DataType.fp32)
    buffer = copy_numpy_to_gpu(np.array([1.0, 2.0], np.float32), stream, DataType.fp32)
    eq = ex.compile(ex.input("x") * ex.tensor_runtime_scalar("step"), device_num=0)
    with pytest.raises(RuntimeError, match="Missing required input tensor: step"):
        eq.stamp({"x": x}, stream)
    with pytest.raises(RuntimeError, match="same dtype as the scalar source dtype"):
        eq.stamp({"x": x}, stream, tensor_scalar_inputs={"step": TensorScalarBinding(buffer, 0, DataType.fp16)})
    with pytest.raises(RuntimeError, match="byte offset is not element-aligned"):
        eq.stamp({"x": x}, stream, tensor_scalar_inputs={"step": TensorScalarBinding(buffer, 2, DataType.fp32)})
    with pytest.raises(RuntimeError, match="exceeds backing buffer size"):
        eq.stamp({"x": x}, stream, tensor_scalar_inputs={"step": TensorScalarBinding(buffer, 8, DataType.fp32)})
    with pytest.raises(RuntimeError, match="Unexpected tensor-runtime-scalar input"):
        eq.stamp({"x": x}, stream, tensor_scalar_inputs={"step": TensorScalarBinding(buffer, 0, DataType.fp32), "other": TensorScalarBinding(buffer, 0, DataType.fp32)})
    with pytest.raises(RuntimeError, match="Input kind mismatch"):
        ex.input("step") * ex.tensor_runtime_scalar("step")
