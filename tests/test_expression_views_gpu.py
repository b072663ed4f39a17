"""Expression::transpose and Expression::stridedView: views of the operand's storage that kernels read through their strides
(reference: Expression.cpp:3769-3787,3854 there), and ragged kernels over such views."""
from __future__ import annotations

import numpy as np
import pytest

from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, gpu_tensor, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def run(outputs, inputs, stream, preallocated=None):
    plan = ex.compile(ex.outputs(outputs), device_num=0).stamp(inputs, stream, preallocated_outputs=preallocated)
    plan.run()
    return plan


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16], ids=lambda d: d.name)
@pytest.mark.parametrize("shape", [(37, 53), (4, 130, 64), (512, 512)], ids=str)
def test_transpose_in_elementwise_work_and_reductions(stream, shape, dtype):
    rng = np.random.default_rng(2)
    x = to_storage(rng.standard_normal(shape).astype(np.float32), dtype)
    y = to_storage(rng.standard_normal(shape[:-2] + (shape[-1], shape[-2])).astype(np.float32), dtype)
    xf, yf = from_storage(x, dtype).astype(np.float64), from_storage(y, dtype).astype(np.float64)
    ix, iy = ex.input("x"), ex.input("y")
    plan = run({"mixed": ix.transpose() * 2.0 + iy, "row_sums": ix.transpose().reduce_sum(axis=len(shape) - 1, squeeze=True),
                "back": (ix.transpose() + iy).transpose() - ix},
               {"x": copy_numpy_to_gpu(x, stream, dtype), "y": copy_numpy_to_gpu(y, stream, dtype)}, stream)
    xt = np.swapaxes(xf, -1, -2)
    tolerance = 1e-5 if dtype == DataType.fp32 else 2e-2
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(plan.output("mixed"), stream), dtype), xt * 2 + yf, rtol=tolerance, atol=tolerance)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("row_sums"), stream).astype(np.float64), xt.sum(axis=-1), rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(plan.output("back"), stream), dtype), np.swapaxes(yf, -1, -2), rtol=tolerance, atol=tolerance)


def test_strided_views_address_the_operands_storage(stream):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((64, 48)).astype(np.float32)
    ix = ex.input("x")
    right_half = ix.strided_view([64, 24], [48, 1], 24)
    diagonal = ix.strided_view([48], [49])
    every_other_row = ix.alias_view([32, 48], [96, 1])
    plan = run({"half": right_half.exp(), "diag": diagonal * 3.0, "rows": every_other_row.reduce_max(axis=0, squeeze=True),
                "of_value": (ix * 2.0).strided_view([64, 8], [48, 1], 40) + 1.0},
               {"x": copy_numpy_to_gpu(x, stream, DataType.fp32)}, stream)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("half"), stream), np.exp(x[:, 24:]), rtol=2e-6)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("diag"), stream), np.diagonal(x)[:48] * np.float32(3))
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("rows"), stream), x[::2].max(axis=0))
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("of_value"), stream), x[:, 40:] * np.float32(2) + np.float32(1))
    with pytest.raises(ValueError, match="one stride per dimension"):
        ix.strided_view([4, 4], [1])
    with pytest.raises(ValueError, match="outside the backing allocation"):
        run({"y": ix.strided_view([64, 48], [48, 2]) + 1.0}, {"x": copy_numpy_to_gpu(x, stream, DataType.fp32)}, stream)
    with pytest.raises(RuntimeError, match="rank 2 or more"):
        run({"y": ex.input("v").transpose() + 1.0}, {"v": copy_numpy_to_gpu(x[0], stream, DataType.fp32)}, stream)


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.bf16], ids=lambda d: d.name)
def test_ragged_kernel_over_a_slice_of_the_packed_values(stream, dtype):
    """A trailing slice [capacity, H] of packed values [capacity, 2H] is a strided view: the kernel is not a flat one, and it
    still stops at the partition's last row (RaggedExpressionTest.cpp:1348-1404 there)."""
    rng = np.random.default_rng(6)
    capacity, width, segments = 900, 32, 5
    x = to_storage(rng.standard_normal((capacity, 2 * width)).astype(np.float32), dtype)
    xf = from_storage(x, dtype)
    offsets = copy_numpy_to_gpu(np.array([0, 100, 100, 350, 351, 700], np.uint32), stream, DataType.uint32)
    values, off = ex.input("x.values"), ex.input("x.offsets")
    gate = values.strided_view([capacity, width], [2 * width, 1], 0)
    up = values.strided_view([capacity, width], [2 * width, 1], width)
    gated = (gate.sigmoid() * up).with_ragged_runtime_extent(off, segments, capacity, width)
    filler = to_storage(np.full((capacity, width), -3.0, np.float32), dtype)
    out = copy_numpy_to_gpu(filler, stream, dtype)
    plan = run({"y": gated}, {"x.values": copy_numpy_to_gpu(x, stream, dtype), "x.offsets": offsets}, stream, {"y": out})
    assert plan.stage_kind_names() == ["FusedKernel"]
    got = from_storage(copy_gpu_to_numpy(out, stream), dtype)
    want = np.full((capacity, width), -3.0, np.float32)
    want[:700] = (1.0 / (1.0 + np.exp(-xf[:700, :width].astype(np.float64)))) * xf[:700, width:]
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-5 if dtype == DataType.fp32 else 3e-2)
    assert np.all(got[700:] == -3.0)
