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


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("offset", [1, 3, 5])
def test_operands_that_begin_inside_a_word_keep_vector_loads(stream, dtype, offset):
    """Views a few elements into their storage, and rows whose pitch no vector divides: the kernels keep their vector length
    and read those operands where they lie; the dense output is written in aligned vectors."""
    rng = np.random.default_rng(offset)
    n = 50_000
    a = to_storage(rng.standard_normal(n + 8).astype(np.float32), dtype)
    b = to_storage(rng.standard_normal(n + 8).astype(np.float32), dtype)
    ta, tb = copy_numpy_to_gpu(a, stream, dtype), copy_numpy_to_gpu(b, stream, dtype)
    va, vb = ta.alias_view([n], [1], element_offset=offset), tb.alias_view([n], [1], element_offset=offset + 1)
    plan = ex.compile(ex.input("a") + ex.input("b"), 0).stamp({"a": va, "b": vb}, stream)
    plan.run()
    assert "vec=1" not in plan.stage_descriptions()[0], plan.stage_descriptions()
    want = to_storage(from_storage(a[offset:offset + n], dtype) + from_storage(b[offset + 1:offset + 1 + n], dtype), dtype)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output(), stream), want)
    # rows of 256 elements cut out of rows of 259: every row begins at another offset inside a word
    m = to_storage(rng.standard_normal((300, 259)).astype(np.float32), dtype)
    c = to_storage(rng.standard_normal(256).astype(np.float32), dtype)
    tm, tc = copy_numpy_to_gpu(m, stream, dtype), copy_numpy_to_gpu(c, stream, dtype)
    vm = tm.alias_view([300, 256], [259, 1], element_offset=offset % 3)
    plan = ex.compile(ex.input("m") * ex.input("c"), 0).stamp({"m": vm, "c": tc}, stream)
    plan.run()
    assert "vec=1" not in plan.stage_descriptions()[0], plan.stage_descriptions()
    rows = m.reshape(-1)[offset % 3:][:299 * 259 + 256]
    window = np.stack([rows[r * 259:r * 259 + 256] for r in range(300)])
    want = to_storage(from_storage(window, dtype) * from_storage(c, dtype), dtype)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output(), stream), want)


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


# ---- take_along_axis (ExpressionConvenienceOpsTest.cpp:357-409 there) ---------------------------------------------------------------
def test_take_along_axis_known_answers(stream):
    values = copy_numpy_to_gpu(np.array([[10, 11, 12, 13], [20, 21, 22, 23]], np.float32), stream, DataType.fp32)
    indices = copy_numpy_to_gpu(np.array([[3, 0, 2], [1, 1, 0]], np.uint32), stream, DataType.uint32)
    plan = run({"y": ex.input("values").take_along_axis(ex.input("indices"))}, {"values": values, "indices": indices}, stream)
    assert plan.output("y").get_dimensions() == [2, 3] and plan.stage_kind_names() == ["FusedKernel"]
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("y"), stream), [[13, 10, 12], [21, 21, 20]])
    values = copy_numpy_to_gpu(np.array([[1, 2], [3, 4], [5, 6]], np.float32), stream, DataType.fp32)
    indices = copy_numpy_to_gpu(np.array([[2, 0], [0, 1]], np.uint32), stream, DataType.uint32)
    plan = run({"y": ex.input("values").take_along_axis(ex.input("indices"), 0)}, {"values": values, "indices": indices}, stream)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("y"), stream), [[5, 2], [1, 4]])


@pytest.mark.parametrize("index_dtype", [DataType.uint32, DataType.uint64], ids=lambda d: d.name)
@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.fp8_e4m3], ids=lambda d: d.name)
@pytest.mark.parametrize("shape,axis,taken", [((7, 50, 33), 1, 9), ((7, 50, 33), 2, 64), ((7, 50, 33), 0, 3), ((4096, 130), -1, 130), ((5,), 0, 11)], ids=str)
def test_take_along_axis_matches_numpy(stream, shape, axis, taken, dtype, index_dtype):
    rng = np.random.default_rng(21)
    x = to_storage(rng.standard_normal(shape).astype(np.float32), dtype)
    index_shape = list(shape)
    index_shape[axis] = taken
    chosen = rng.integers(0, shape[axis], index_shape).astype(np.uint32 if index_dtype == DataType.uint32 else np.uint64)
    plan = run({"y": ex.input("x").take_along_axis(ex.input("i"), axis)}, {"x": copy_numpy_to_gpu(x, stream, dtype), "i": copy_numpy_to_gpu(chosen, stream, index_dtype)},
               stream)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("y"), stream), np.take_along_axis(x, chosen.astype(np.int64), axis))  # a copy: bit-exact


def test_take_along_axis_of_computed_operands(stream):
    rng = np.random.default_rng(22)
    x = rng.standard_normal((300, 77)).astype(np.float32)
    ix = ex.input("x")
    # the value at the row's argmax is the row's max; a transposed operand is gathered from a dense copy
    outputs = {"at_argmax": (ix * 2.0).take_along_axis(ix.argmax(axis=1), 1), "row_max": ix.reduce_max(axis=1) * 2.0,
               "of_transpose": ix.transpose().take_along_axis(ix.transpose().argmin(axis=0), 0)}
    plan = run(outputs, {"x": copy_numpy_to_gpu(x, stream, DataType.fp32)}, stream)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("at_argmax"), stream), copy_gpu_to_numpy(plan.output("row_max"), stream))
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("of_transpose"), stream), x.min(axis=1)[None, :])
    # indices past the end read the last element of the axis instead of leaving the tensor
    far = copy_numpy_to_gpu(np.full((300, 2), 1000, np.uint32), stream, DataType.uint32)
    plan = run({"y": ix.take_along_axis(ex.input("i"))}, {"x": copy_numpy_to_gpu(x, stream, DataType.fp32), "i": far}, stream)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("y"), stream), np.repeat(x[:, -1:], 2, axis=1))


def test_take_along_axis_validation(stream):
    x = copy_numpy_to_gpu(np.zeros((4, 6), np.float32), stream, DataType.fp32)
    ix, ii = ex.input("x"), ex.input("i")
    with pytest.raises(RuntimeError, match="indices must have UINT32 or UINT64 dtype, received"):
        run({"y": ix.take_along_axis(ii)}, {"x": x, "i": x}, stream)
    with pytest.raises(RuntimeError, match="must have the same rank"):
        run({"y": ix.take_along_axis(ii)}, {"x": x, "i": copy_numpy_to_gpu(np.zeros((4,), np.uint32), stream, DataType.uint32)}, stream)
    with pytest.raises(RuntimeError, match="must match except on the selected axis"):
        run({"y": ix.take_along_axis(ii, 1)}, {"x": x, "i": copy_numpy_to_gpu(np.zeros((3, 2), np.uint32), stream, DataType.uint32)}, stream)
    with pytest.raises(RuntimeError, match="axis is out of range"):
        run({"y": ix.take_along_axis(ii, 2)}, {"x": x, "i": copy_numpy_to_gpu(np.zeros((4, 2), np.uint32), stream, DataType.uint32)}, stream)
    with pytest.raises(ValueError, match="only axis=-1 or an explicit non-negative axis"):
        ix.take_along_axis(ii, -2)


# ---- backward of strided views: the gradient lands on the elements the view addresses ---------------------------------------------
@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16], ids=lambda d: d.name)
def test_gradient_through_slices_of_one_input(stream, dtype):
    rng = np.random.default_rng(41)
    x = to_storage(rng.uniform(-1, 1, (300, 24)).astype(np.float32), dtype)
    g = to_storage(rng.uniform(-1, 1, (300, 12)).astype(np.float32), dtype)
    ix = ex.input("x")
    gate, value = ix.strided_view([300, 12], [24, 1], 12), ix.strided_view([300, 12], [24, 1], 0)
    fwd = ex.compile(gate.tanh() * value, device_num=0)
    plan = fwd.compile_backward(["x"], error_input_name="__grad_output").stamp(
        {"x": copy_numpy_to_gpu(x, stream, dtype), "__grad_output": copy_numpy_to_gpu(g, stream, dtype)}, stream)
    plan.run()
    assert sum("view_scatter" in d for d in plan.stage_descriptions()) == 2 and plan.output("x_grad").get_data_type() == dtype
    xf, gf = from_storage(x, dtype).astype(np.float64), from_storage(g, dtype).astype(np.float64)
    expected = np.concatenate([gf * np.tanh(xf[:, 12:]), gf * (1 - np.tanh(xf[:, 12:]) ** 2) * xf[:, :12]], axis=1)
    tolerance = 2e-6 if dtype == DataType.fp32 else 4e-3
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(plan.output("x_grad"), stream), dtype), expected, rtol=tolerance, atol=tolerance)


def test_gradient_of_permuted_and_strided_views(stream):
    rng = np.random.default_rng(42)
    x = rng.standard_normal((6, 10, 8)).astype(np.float32)
    g = rng.standard_normal((8, 5, 3)).astype(np.float32)
    # every second row of the last three planes, axes reversed: view[c, r, p] = x[3 + p, 2 r, c]
    view = ex.input("x").strided_view([8, 5, 3], [1, 16, 80], 240)
    plan = ex.compile(view * 2.0, device_num=0).compile_backward(["x"], error_input_name="__grad_output").stamp(
        {"x": copy_numpy_to_gpu(x, stream, DataType.fp32), "__grad_output": copy_numpy_to_gpu(g, stream, DataType.fp32)}, stream)
    plan.run()
    expected = np.zeros_like(x)
    expected[3:, ::2, :] = 2.0 * np.transpose(g, (2, 1, 0))
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("x_grad"), stream), expected)
    # a view that reads an element twice has no gradient here, nor has a view of a view
    tensors = {"x": copy_numpy_to_gpu(x, stream, DataType.fp32)}
    with pytest.raises(RuntimeError, match="addresses every element once"):
        ex.compile(ex.input("x").strided_view([4, 100], [50, 1], 0) * 2.0, device_num=0).compile_backward(["x"]).stamp(tensors, stream)
    with pytest.raises(RuntimeError, match="operand is itself a view"):
        ex.compile(ex.input("x").transpose().strided_view([4, 4], [8, 1], 0) * 2.0, device_num=0).compile_backward(["x"]).stamp(tensors, stream)
