"""Expression.scan / segmented_scan / prefix_count and their backward equations, with the literal cases of the reference's
bindings/python/test/core/physical/test_expression_scan.py, test_expression_arg_scan.py, test_expression_mask_scan.py,
test_expression_segmented_scan.py and test_expression_backward_phase1.py:73-113."""
from __future__ import annotations

import numpy as np
import pytest

import oracle
from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex, ScanOp

pytestmark = pytest.mark.gpu
ORACLE_OP = {ScanOp.sum: oracle.SCAN_SUM, ScanOp.min: oracle.SCAN_MIN, ScanOp.max: oracle.SCAN_MAX, ScanOp.product: oracle.SCAN_PRODUCT,
             ScanOp.arg_min: oracle.SCAN_ARGMIN, ScanOp.arg_max: oracle.SCAN_ARGMAX}


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def stamp_run(outputs, tensors, stream):
    plan = ex.compile(ex.outputs(outputs) if isinstance(outputs, dict) else outputs, device_num=0).stamp(tensors, stream)
    plan.run()
    return plan


@pytest.mark.parametrize("inclusive", [True, False])
@pytest.mark.parametrize("op", [ScanOp.sum, ScanOp.min, ScanOp.max, ScanOp.product])
def test_scan_expression_matches_numpy_reference(stream, op, inclusive):
    values = np.array([[2, 3, 1, 4], [5, 1, 2, 3]], np.uint32)
    plan = stamp_run(ex.input("x").scan(op=op, axis=-1, inclusive=inclusive), {"x": copy_numpy_to_gpu(values, stream, DataType.uint32)}, stream)
    assert plan.stage_kind_names() == ["Scan"]
    assert plan.output().get_data_type() == DataType.uint32
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output(), stream), oracle.scan(values, ORACLE_OP[op], inclusive, segment_size=4, dtype=oracle.UINT32))


@pytest.mark.parametrize("inclusive", [True, False])
@pytest.mark.parametrize("name", ["min", "max"])
def test_scan_with_indices_returns_values_and_flattened_winner_indices(stream, name, inclusive):
    values = np.array([[3.0, 1.0, 4.0, 1.0], [2.0, 5.0, 0.0, 0.0]], np.float32)
    found, indices = ex.input("x").scan_with_indices(op=ScanOp[name], axis=-1, inclusive=inclusive)
    plan = stamp_run({"values": found, "indices": indices}, {"x": copy_numpy_to_gpu(values, stream, DataType.fp32)}, stream)
    assert plan.stage_kind_names() == ["Scan"]  # values and indices come from one pass
    expected_indices = oracle.scan(values, ORACLE_OP[ScanOp["arg_" + name]], inclusive, segment_size=4)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("indices"), stream), expected_indices)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("values"), stream), oracle.scan(values, ORACLE_OP[ScanOp[name]], inclusive, segment_size=4))
    if inclusive:  # [[0, 1, 1, 1], [4, 4, 6, 6]] for min: the first of two equal values wins
        assert expected_indices.tolist() == ([[0, 1, 1, 1], [4, 4, 6, 6]] if name == "min" else [[0, 0, 2, 2], [4, 5, 5, 5]])


@pytest.mark.parametrize("offsets_dtype", [DataType.uint32, DataType.uint64], ids=lambda d: d.name)
@pytest.mark.parametrize("inclusive", [True, False])
@pytest.mark.parametrize("op", [ScanOp.sum, ScanOp.min, ScanOp.max, ScanOp.product, ScanOp.arg_min, ScanOp.arg_max], ids=lambda o: o.name)
def test_segmented_scan_expression(stream, op, inclusive, offsets_dtype):
    values = np.array([8, 6, 7, 5, 3, 2, 9], np.uint32)
    offsets = np.array([0, 2, 5, 7], np.uint32 if offsets_dtype == DataType.uint32 else np.uint64)
    plan = stamp_run(ex.input("x").segmented_scan(ex.input("offsets"), op=op, inclusive=inclusive),
                     {"x": copy_numpy_to_gpu(values, stream, DataType.uint32), "offsets": copy_numpy_to_gpu(offsets, stream, offsets_dtype)}, stream)
    assert plan.stage_kind_names() == ["Scan"]
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output(), stream), oracle.scan(values, ORACLE_OP[op], inclusive, offsets=offsets, dtype=oracle.UINT32))


def test_bool_mask_prefix_count(stream):
    values = np.array([[0.0, 2.0, -1.0, 3.0], [4.0, -5.0, 6.0, 7.0]], np.float32)
    x = ex.input("x")
    mask = x > 0.0
    plan = stamp_run({"inclusive": mask.prefix_count(inclusive=True, axis=-1), "exclusive": mask.prefix_count(inclusive=False, axis=-1),
                      "direct": (x != 0.0).cast(DataType.uint32).scan(op=ScanOp.sum)}, {"x": copy_numpy_to_gpu(values, stream, DataType.fp32)}, stream)
    counts = np.cumsum((values > 0).astype(np.uint32), axis=-1, dtype=np.uint32)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("inclusive"), stream), counts)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("exclusive"), stream), np.concatenate([np.zeros((2, 1), np.uint32), counts[:, :-1]], axis=1))
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("direct"), stream), np.cumsum((values != 0).astype(np.uint32), axis=-1, dtype=np.uint32))


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
def test_scans_inside_larger_expressions(stream, dtype):
    """A running maximum subtracted from the input, a cumulative sum of a computed operand, the scan of a transposed operand."""
    rng = np.random.default_rng(51)
    x = to_storage((np.round(rng.standard_normal((200, 96)) * 8) / 8).astype(np.float32), dtype)
    xf = from_storage(x, dtype).astype(np.float64)
    ix = ex.input("x")
    outputs = {"drawdown": ix - ix.scan(ScanOp.max), "energy": (ix * ix).scan(ScanOp.sum), "of_transpose": ix.transpose().scan(ScanOp.min, reverse=True)}
    plan = stamp_run(outputs, {"x": copy_numpy_to_gpu(x, stream, dtype)}, stream)
    tolerance = 1e-5 if dtype == DataType.fp32 else 4e-2
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(plan.output("drawdown"), stream), dtype), xf - np.maximum.accumulate(xf, axis=1), atol=tolerance)
    squares = from_storage(to_storage((xf * xf).astype(np.float32), dtype), dtype).astype(np.float64) if dtype != DataType.fp32 else xf * xf
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(plan.output("energy"), stream), dtype), np.cumsum(squares, axis=1), rtol=tolerance, atol=tolerance)
    np.testing.assert_array_equal(from_storage(copy_gpu_to_numpy(plan.output("of_transpose"), stream), dtype),
                                  np.minimum.accumulate(xf.T[:, ::-1], axis=1)[:, ::-1].astype(np.float32))


# ---- backward: the gradient of a sum scan is the same scan from the other end ------------------------------------------------
@pytest.mark.parametrize("inclusive", [True, False])
@pytest.mark.parametrize("dtype", [DataType.fp16, DataType.bf16, DataType.fp32], ids=lambda d: d.name)
def test_sum_scan_backward_is_a_reverse_scan(stream, dtype, inclusive):
    x = to_storage(np.array([[1.0, 2.0, 3.0, 4.0], [1.5, -0.5, 2.5, 0.25]], np.float32), dtype)
    g = to_storage(np.array([[0.5, -1.0, 0.25, 2.0], [1.25, 0.75, -0.5, 1.5]], np.float32), dtype)
    bwd = ex.compile(ex.input("x").scan(ScanOp.sum, axis=-1, inclusive=inclusive), device_num=0).compile_backward(["x"], error_input_name="__grad_output")
    plan = bwd.stamp({"x": copy_numpy_to_gpu(x, stream, dtype), "__grad_output": copy_numpy_to_gpu(g, stream, dtype)}, stream)
    assert plan.stage_kind_names() == ["Scan"]
    plan.run()
    gf = from_storage(g, dtype).astype(np.float64)
    reverse = np.flip(np.cumsum(np.flip(gf, axis=-1), axis=-1), axis=-1)
    expected = reverse if inclusive else np.concatenate([reverse[:, 1:], np.zeros((2, 1))], axis=1)
    tolerance = {DataType.fp32: (1e-5, 1e-6), DataType.fp16: (5e-2, 5e-2), DataType.bf16: (5e-2, 5e-2)}[dtype]
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(plan.output("x_grad"), stream), dtype), expected, rtol=tolerance[0], atol=tolerance[1])


@pytest.mark.parametrize("offsets_dtype", [DataType.uint32, DataType.uint64], ids=lambda d: d.name)
@pytest.mark.parametrize("inclusive", [True, False])
def test_segmented_sum_scan_backward_uses_ragged_reverse_scan(stream, inclusive, offsets_dtype):
    x = np.array([1.0, 2.0, 3.0, 4.0, -1.0, 0.5, 2.5], np.float32)
    g = np.array([0.5, -1.0, 0.25, 2.0, 1.25, -0.5, 1.5], np.float32)
    offsets = np.array([0, 3, 3, 7], np.uint32 if offsets_dtype == DataType.uint32 else np.uint64)
    forward = ex.input("x").segmented_scan(ex.input("offsets"), op=ScanOp.sum, inclusive=inclusive)
    bwd = ex.compile(forward, device_num=0).compile_backward(["x"], error_input_name="__grad_output")
    assert bwd.output_names() == ["x_grad"]
    plan = bwd.stamp({"x": copy_numpy_to_gpu(x, stream, DataType.fp32), "offsets": copy_numpy_to_gpu(offsets, stream, offsets_dtype),
                      "__grad_output": copy_numpy_to_gpu(g, stream, DataType.fp32)}, stream)
    assert plan.stage_kind_names() == ["Scan"]
    plan.run()
    expected = np.empty_like(g)
    for s in range(3):
        begin, end = int(offsets[s]), int(offsets[s + 1])
        rev = g[begin:end][::-1]
        inc = np.cumsum(rev)
        expected[begin:end] = (inc if inclusive else np.concatenate([[0.0], inc[:-1]])[: len(rev)])[::-1]
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("x_grad"), stream), expected, rtol=1e-5, atol=1e-6)
    with pytest.raises(RuntimeError, match="offsets are metadata and are not differentiable"):
        ex.compile(forward, device_num=0).compile_backward(["offsets"], error_input_name="__grad_output").stamp(
            {"x": copy_numpy_to_gpu(x, stream, DataType.fp32), "offsets": copy_numpy_to_gpu(offsets, stream, offsets_dtype),
             "__grad_output": copy_numpy_to_gpu(g, stream, DataType.fp32)}, stream)


def test_scan_inside_a_loss_has_the_right_gradient(stream):
    rng = np.random.default_rng(53)
    values = rng.uniform(-1, 1, (40, 33)).astype(np.float32)
    weights = rng.uniform(-1, 1, (40, 33)).astype(np.float32)
    x, w = ex.input("x"), ex.input("w")
    loss = (x.exp().scan(ScanOp.sum, inclusive=False) * w).reduce_sum(axis=[0, 1])
    bwd = ex.compile(loss, device_num=0).compile_backward(["x"])
    plan = bwd.stamp({"x": copy_numpy_to_gpu(values, stream, DataType.fp32), "w": copy_numpy_to_gpu(weights, stream, DataType.fp32)}, stream)
    plan.run()
    # d/dx_j sum_i w_i * sum_{k<i} e^{x_k} = e^{x_j} * sum_{i>j} w_i
    later = np.flip(np.cumsum(np.flip(weights.astype(np.float64), axis=1), axis=1), axis=1) - weights
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("x_grad"), stream), np.exp(values.astype(np.float64)) * later, rtol=2e-5, atol=2e-6)


def test_validation(stream):
    x = copy_numpy_to_gpu(np.zeros((4, 6), np.float32), stream, DataType.fp32)
    ix = ex.input("x")
    with pytest.raises(RuntimeError, match="only axis=-1 or an explicit non-negative final axis"):
        stamp_run(ix.scan(ScanOp.sum, axis=0), {"x": x}, stream)
    with pytest.raises(ValueError, match="only axis=-1 or an explicit non-negative final axis"):
        ix.scan(ScanOp.sum, axis=-2)
    with pytest.raises(RuntimeError, match="requires UINT32, FP16, BF16 or FP32 values"):
        stamp_run(ix.scan(ScanOp.sum), {"x": copy_numpy_to_gpu(np.zeros((4, 6), np.int32), stream, DataType.int32)}, stream)
    with pytest.raises(RuntimeError, match="offsets must have UINT32 or UINT64 dtype"):
        stamp_run(ex.input("v").segmented_scan(ex.input("o")), {"v": copy_numpy_to_gpu(np.zeros(6, np.float32), stream, DataType.fp32),
                                                                "o": copy_numpy_to_gpu(np.zeros(3, np.float32), stream, DataType.fp32)}, stream)
    with pytest.raises(ValueError, match="supports only ScanOp.min and ScanOp.max"):
        ix.scan_with_indices(ScanOp.sum)
    with pytest.raises(RuntimeError, match="supports backward only for sum/min/max scan"):
        ex.compile(ix.scan(ScanOp.product), device_num=0).compile_backward(["x"]).stamp({"x": x}, stream)
    stamp_run(ix.scan(ScanOp.sum, axis=1), {"x": x}, stream)  # the index of the last axis is accepted


@pytest.mark.parametrize("inclusive", [True, False])
@pytest.mark.parametrize("name", ["min", "max"])
def test_segmented_scan_with_indices_is_one_stage(stream, name, inclusive):
    """test_expression_arg_scan.py:180-228 there."""
    values = np.array([8, 6, 7, 5, 3, 2, 9], np.uint32)
    offsets = np.array([0, 2, 5, 7], np.uint32)
    found, indices = ex.input("x").segmented_scan_with_indices(ex.input("offsets"), op=ScanOp[name], inclusive=inclusive)
    plan = stamp_run({"values": found, "indices": indices},
                     {"x": copy_numpy_to_gpu(values, stream, DataType.uint32), "offsets": copy_numpy_to_gpu(offsets, stream, DataType.uint32)}, stream)
    assert plan.stage_kind_names() == ["Scan"]
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("values"), stream), oracle.scan(values, ORACLE_OP[ScanOp[name]], inclusive, offsets=offsets, dtype=oracle.UINT32))
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("indices"), stream),
                                  oracle.scan(values, ORACLE_OP[ScanOp["arg_" + name]], inclusive, offsets=offsets, dtype=oracle.UINT32))


# ---- min / max scans backward: every position's gradient goes to the element that held the running extreme there -----------------
MINMAX_BACKWARD_EXPECTED = {  # worked out by hand for the vectors of test_segmented_minmax_scan_backward_uses_arg_scan_and_flat_scatter_add there
    ("min", True): [0.5, -0.75, 0.0, 2.0, 0.75, 0.0, 1.5], ("max", True): [-0.25, 0.0, 0.0, 4.25, 0.0, 0.0, 0.0],
    ("min", False): [-1.0, 0.25, 0.0, 1.25, 1.0, 0.0, 0.0], ("max", False): [-0.75, 0.0, 0.0, 2.25, 0.0, 0.0, 0.0]}


@pytest.mark.parametrize("dtype", [DataType.fp16, DataType.bf16, DataType.fp32], ids=lambda d: d.name)
@pytest.mark.parametrize("inclusive", [True, False])
@pytest.mark.parametrize("name", ["min", "max"])
def test_segmented_minmax_scan_backward_uses_arg_scan_and_scatter_add(stream, name, inclusive, dtype):
    values = to_storage(np.array([3.0, 1.0, 1.0, 4.0, 2.0, 2.0, 0.0], np.float32), dtype)
    grad = to_storage(np.array([0.5, -1.0, 0.25, 2.0, 1.25, -0.5, 1.5], np.float32), dtype)
    offsets = np.array([0, 3, 3, 7], np.uint32)
    fwd = ex.compile(ex.input("x").segmented_scan(ex.input("offsets"), op=ScanOp[name], inclusive=inclusive), device_num=0)
    bwd = fwd.compile_backward(["x"], error_input_name="__grad_output")
    assert bwd.output_names() == ["x_grad"]
    plan = bwd.stamp({"x": copy_numpy_to_gpu(values, stream, dtype), "offsets": copy_numpy_to_gpu(offsets, stream, DataType.uint32),
                      "__grad_output": copy_numpy_to_gpu(grad, stream, dtype)}, stream)
    plan.run()
    assert plan.stage_kind_names().count("Scan") == 1 and sum("scatter_add" in d for d in plan.stage_descriptions()) == 1
    assert plan.output("x_grad").get_data_type() == dtype
    got = from_storage(copy_gpu_to_numpy(plan.output("x_grad"), stream), dtype)
    np.testing.assert_allclose(got, MINMAX_BACKWARD_EXPECTED[(name, inclusive)], rtol=1e-5, atol=1e-6)


def winners_gradient(values, grad, op, inclusive, reverse=False, segment_size=0, offsets=None, dtype=oracle.FP32):
    """Scatter of `grad` by the oracle's arg scan, in float64."""
    winners = oracle.scan(values, op, inclusive, reverse, segment_size=segment_size, offsets=offsets, dtype=dtype).reshape(-1)
    live = np.ones(winners.size, bool)
    if offsets is not None:
        live[:] = False
        live[int(offsets[0]):int(offsets[-1])] = True
    live &= winners != 0xFFFFFFFF
    expected = np.zeros(winners.size, np.float64)
    np.add.at(expected, winners[live].astype(np.int64), grad.reshape(-1).astype(np.float64)[live])
    return expected.reshape(values.shape)


# Every shape meets every (inclusive, reverse) pair in fp32, min and max taking turns; bf16 meets every shape once, with the
# other operation, and every pair at least once.
ROUTE_SHAPES = [(64, 1000), (3, 20000), (1, 7), (16, 8192), (300, 256), (37, 33), (9, 4100)]
ROUTE_MODES = [(True, False), (False, False), (True, True), (False, True)]
ROUTE_CASES = [(s, ("min", "max")[(i + j) % 2], m[0], m[1], DataType.fp32) for i, s in enumerate(ROUTE_SHAPES) for j, m in enumerate(ROUTE_MODES)]
ROUTE_CASES += [(s, ("max", "min")[i % 2], *ROUTE_MODES[i % 4], DataType.bf16) for i, s in enumerate(ROUTE_SHAPES)]


@pytest.mark.parametrize("shape,name,inclusive,reverse,dtype", ROUTE_CASES,
                         ids=[f"{s}-{n}-{'incl' if i else 'excl'}{'-rev' if r else ''}-{d.name}" for s, n, i, r, d in ROUTE_CASES])
def test_row_minmax_scan_backward(stream, shape, name, inclusive, reverse, dtype):
    rng = np.random.default_rng(61)
    # few distinct values: long runs of one winner, and ties that the first occurrence must win
    values = to_storage(rng.integers(-6, 7, shape).astype(np.float32) * 0.5, dtype)
    grad = to_storage(rng.integers(-8, 9, shape).astype(np.float32) * 0.25, dtype)  # sums of these are exact in fp32
    ix = ex.input("x")
    scanned = ix.scan(ScanOp[name], inclusive=inclusive, reverse=reverse)
    bwd = ex.compile(scanned, device_num=0).compile_backward(["x"], error_input_name="__grad_output")
    plan = bwd.stamp({"x": copy_numpy_to_gpu(values, stream, dtype), "__grad_output": copy_numpy_to_gpu(grad, stream, dtype)}, stream)
    plan.run()
    # rows that fit one block's chunk (8192 positions) take one launch: winners, run sums and the routed gradient together
    descriptions = " | ".join(plan.stage_descriptions())
    assert ("scan-route" in descriptions) == (shape[-1] <= 8192) and ("scatter_add" in descriptions) == (shape[-1] > 8192), descriptions
    expected = winners_gradient(values, from_storage(grad, dtype), ORACLE_OP[ScanOp["arg_" + name]], inclusive, reverse, segment_size=shape[-1], dtype=int(dtype))
    got = from_storage(copy_gpu_to_numpy(plan.output("x_grad"), stream), dtype).astype(np.float64)
    if dtype == DataType.fp32:
        np.testing.assert_array_equal(got, expected)  # exact sums: the order of the additions cannot show
    else:
        np.testing.assert_allclose(got, from_storage(to_storage(expected.astype(np.float32), dtype), dtype), rtol=0, atol=0)


def test_row_running_max_backward_with_real_gradients(stream):
    """Random fp32 gradients: the run sums are compared with float64 sums within the rounding of a tree of fp32 additions, and
    every element that never held the running maximum gets exactly zero."""
    rng = np.random.default_rng(63)
    values = rng.standard_normal((256, 8192)).astype(np.float32)
    grad = rng.standard_normal((256, 8192)).astype(np.float32)
    bwd = ex.compile(ex.input("x").scan(ScanOp.max), device_num=0).compile_backward(["x"], error_input_name="__grad_output")
    plan = bwd.stamp({"x": copy_numpy_to_gpu(values, stream, DataType.fp32), "__grad_output": copy_numpy_to_gpu(grad, stream, DataType.fp32)}, stream)
    assert plan.stage_kind_names() == ["Scan"]
    for _ in range(2):  # the LDS copy is cleared by every launch
        plan.run()
        got = copy_gpu_to_numpy(plan.output("x_grad"), stream).astype(np.float64)
        expected = winners_gradient(values, grad, oracle.SCAN_ARGMAX, True, segment_size=8192)
        scale = np.zeros_like(expected)
        winners = oracle.scan(values, oracle.SCAN_ARGMAX, True, segment_size=8192, dtype=oracle.FP32).reshape(-1).astype(np.int64)
        np.add.at(scale.reshape(-1), winners, np.abs(grad.reshape(-1)).astype(np.float64))
        assert np.all(np.abs(got - expected) <= 2e-6 * scale)
        assert np.all(got[scale == 0] == 0)


def test_ragged_minmax_scan_backward_and_chain_rule(stream):
    rng = np.random.default_rng(62)
    n = 50_000
    cuts = np.sort(rng.choice(np.arange(1, n - 500), 300, replace=False))
    offsets = np.concatenate([[0], cuts, [n - 500]]).astype(np.uint64)  # the last 500 values belong to no segment
    values = (rng.integers(-50, 51, n).astype(np.float32)) * 0.125
    grad = rng.integers(-8, 9, n).astype(np.float32) * 0.25
    v, o = ex.input("v"), ex.input("o")
    fwd = ex.compile(v.segmented_scan(o, ScanOp.max, inclusive=True, reverse=True), device_num=0)
    plan = fwd.compile_backward(["v"], error_input_name="__grad_output").stamp(
        {"v": copy_numpy_to_gpu(values, stream, DataType.fp32), "o": copy_numpy_to_gpu(offsets, stream, DataType.uint64),
         "__grad_output": copy_numpy_to_gpu(grad, stream, DataType.fp32)}, stream)
    plan.run()
    expected = winners_gradient(values, grad, oracle.SCAN_ARGMAX, True, True, offsets=offsets)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("v_grad"), stream), expected)
    assert np.all(expected[n - 500:] == 0)
    # through elementwise work on both sides: d/dx sum(w * cummax(x^2)) = 2 x * scatter(w)
    x32 = rng.uniform(0.5, 2.0, (30, 257)).astype(np.float32)
    w32 = rng.integers(-4, 5, (30, 257)).astype(np.float32)
    x, w = ex.input("x"), ex.input("w")
    loss = ((x * x).scan(ScanOp.max) * w).reduce_sum(axis=[0, 1])
    plan = ex.compile(loss, device_num=0).compile_backward(["x"]).stamp({"x": copy_numpy_to_gpu(x32, stream, DataType.fp32), "w": copy_numpy_to_gpu(w32, stream, DataType.fp32)},
                                                                        stream)
    plan.run()
    squares = x32 * x32
    expected = 2.0 * x32.astype(np.float64) * winners_gradient(squares, w32, oracle.SCAN_ARGMAX, True, segment_size=257)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("x_grad"), stream), expected, rtol=1e-6, atol=1e-6)
