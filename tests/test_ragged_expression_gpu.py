"""Ragged-batch Expression ops (segmented reductions, segmented broadcast, runtime-extent kernels) through compile / stamp / run,
with the reference's RaggedExpressionTest.cpp execution cases as known answers and numpy loops over the segments otherwise."""
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


class Ragged:
    """The composition rules of the reference's RaggedExpression (RaggedExpression.cpp:204-330) spelled with Expression primitives."""

    def __init__(self, name, batch, capacity, trailing=()):
        self.values, self.offsets = ex.input(name + ".values"), ex.input(name + ".offsets")
        self.batch, self.capacity, self.trailing = batch, capacity, tuple(trailing)
        self.elements = int(np.prod(trailing)) if trailing else 1

    def wrap(self, values):
        return values.with_ragged_runtime_extent(self.offsets, self.batch, self.capacity, self.elements)

    def reduce(self, values, kind):
        return getattr(values, "segment_" + kind)(self.offsets, self.batch, self.capacity, self.elements)

    def spread(self, per_segment, normalize=False):
        return per_segment.segmented_broadcast(self.offsets, self.batch, self.capacity, self.elements, normalize)

    def softmax(self, log=False):
        shifted = self.values - self.spread(self.reduce(self.values, "max"))
        e = shifted.exp()
        total = self.spread(self.reduce(e, "sum"))
        return self.wrap(shifted - total.ln() if log else e / total)


def run(expr_or_outputs, inputs, stream, preallocated=None):
    eq = ex.compile(expr_or_outputs, device_num=0)
    plan = eq.stamp(inputs, stream, preallocated_outputs=preallocated)
    plan.run()
    return plan, eq


def test_segment_sum_min_max_mean_for_empty_and_skewed_rows(stream):
    """RaggedExpressionTest.cpp:1795-1824."""
    r = Ragged("x", 4, 9)
    inputs = {"x.values": copy_numpy_to_gpu(np.array([1, -2, 4, 5, 7, -1, 8, 99, 100], np.float32), stream, DataType.fp32),
              "x.offsets": copy_numpy_to_gpu(np.array([0, 3, 3, 5, 7], np.uint32), stream, DataType.uint32)}
    outputs = ex.outputs({k: r.reduce(r.values, k) for k in ("sum", "min", "max", "mean")})
    plan, eq = run(outputs, inputs, stream)
    assert sorted(plan.stage_kind_names()) == ["SegmentedReduction"] * 4
    got = {k: copy_gpu_to_numpy(plan.output(k), stream) for k in ("sum", "min", "max", "mean")}
    np.testing.assert_array_equal(got["sum"], np.array([3, 0, 12, 7], np.float32))
    np.testing.assert_array_equal(got["mean"], np.array([1, 0, 6, 3.5], np.float32))
    np.testing.assert_array_equal(got["min"], np.array([-2, np.inf, 5, -1], np.float32))
    np.testing.assert_array_equal(got["max"], np.array([4, -np.inf, 7, 8], np.float32))


@pytest.mark.parametrize("log", [False, True], ids=["softmax", "log_softmax"])
def test_segment_softmax_per_row_leaves_unused_capacity_untouched(stream, log):
    """RaggedExpressionTest.cpp:1826-1884: scalar values, an empty row, three rows of capacity nobody owns."""
    r = Ragged("x", 3, 8)
    x = np.array([1, 2, 0, -1, 1, 50, 60, 70], np.float32)
    inputs = {"x.values": copy_numpy_to_gpu(x, stream, DataType.fp32), "x.offsets": copy_numpy_to_gpu(np.array([0, 2, 2, 5], np.uint32), stream, DataType.uint32)}
    out = copy_numpy_to_gpu(np.full(8, 321.0, np.float32), stream, DataType.fp32)
    plan, _ = run(ex.outputs({"y": r.softmax(log)}), inputs, stream, {"y": out})
    got = copy_gpu_to_numpy(plan.output("y"), stream)
    want = np.full(8, 321.0, np.float64)
    for lo, hi in ((0, 2), (2, 5)):
        e = np.exp(x[lo:hi].astype(np.float64) - x[lo:hi].max())
        want[lo:hi] = np.log(e / e.sum()) if log else e / e.sum()
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-5)
    assert np.array_equal(got[5:], np.full(3, 321.0, np.float32))


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.bf16, DataType.fp16], ids=lambda d: d.name)
def test_vector_segment_softmax_per_component(stream, dtype):
    """RaggedExpressionTest.cpp:1940-1981: [32, 2] capacity, five active rows in four segments, fp16 / bf16 / fp32."""
    capacity = 32
    values = np.full((capacity, 2), 91.0, np.float32)
    values[:5] = np.array([[1, 10], [3, 6], [-1, 4], [5, -2], [7, 8]], np.float32)
    r = Ragged("x", 4, capacity, (2,))
    inputs = {"x.values": copy_numpy_to_gpu(to_storage(values, dtype), stream, dtype),
              "x.offsets": copy_numpy_to_gpu(np.array([0, 2, 2, 3, 5], np.uint32), stream, DataType.uint32)}
    out = copy_numpy_to_gpu(to_storage(np.full((capacity, 2), 77.0, np.float32), dtype), stream, dtype)
    plan, _ = run(ex.outputs({"y": r.softmax()}), inputs, stream, {"y": out})
    got = from_storage(copy_gpu_to_numpy(plan.output("y"), stream), dtype)
    e2, e10, e6 = np.exp(2.0), np.exp(10.0), np.exp(6.0)
    want = np.full((capacity, 2), 77.0)
    want[:5] = [[1 / (1 + e2), e10 / (e10 + e6)], [e2 / (1 + e2), e6 / (e10 + e6)], [1, 1], [1 / (1 + e2), 1 / (1 + e10)], [e2 / (1 + e2), e10 / (1 + e10)]]
    np.testing.assert_allclose(got, want, rtol=0, atol=3e-5 if dtype == DataType.fp32 else 2e-2)


def test_valuewise_kernels_follow_the_offsets_of_each_run(stream):
    """RaggedExpressionTest.cpp:1758-1793: the active extent is read on the device, so one stamped plan serves every partition."""
    r = Ragged("x", 3, 1000, (3,))
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1000, 3)).astype(np.float32)
    offsets = copy_numpy_to_gpu(np.array([0, 10, 10, 40], np.uint32), stream, DataType.uint32)
    inputs = {"x.values": copy_numpy_to_gpu(x, stream, DataType.fp32), "x.offsets": offsets}
    out = gpu_tensor([1000, 3], DataType.fp32)
    plan, _ = run(ex.outputs({"y": r.wrap((r.values * 2.0 + 1.0).abs())}), inputs, stream, {"y": out})
    assert plan.stage_kind_names() == ["FusedKernel"]
    for active in (40, 7, 1000, 0, 333):
        out.copy_from_async(copy_numpy_to_gpu(np.full((1000, 3), -5.0, np.float32), stream, DataType.fp32), stream)
        offsets.copy_from_async(copy_numpy_to_gpu(np.array([0, min(active, 3), min(active, 3), active], np.uint32), stream, DataType.uint32), stream)
        plan.run()
        got = copy_gpu_to_numpy(out, stream)
        np.testing.assert_array_equal(got[:active], np.abs(x[:active] * np.float32(2.0) + np.float32(1.0)))
        assert np.all(got[active:] == -5.0), active


SHAPES = [((5000,), 37), ((4096, 8), 300), ((3000, 3, 5), 12), ((20000, 64), 2000)]


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("shape,segments", SHAPES, ids=[f"{s}-{b}" for s, b in SHAPES])
def test_random_ragged_softmax_and_centering_against_numpy(stream, shape, segments, dtype):
    rng = np.random.default_rng(segments)
    capacity = shape[0]
    active = capacity - capacity // 5
    cuts = np.sort(rng.integers(0, active + 1, segments - 1))
    offsets = np.concatenate([[0], cuts, [active]]).astype(np.int64)
    x = to_storage(rng.standard_normal(shape).astype(np.float32) * 3, dtype)
    xf = from_storage(x, dtype).astype(np.float64)
    r = Ragged("x", segments, capacity, shape[1:])
    inputs = {"x.values": copy_numpy_to_gpu(x, stream, dtype), "x.offsets": copy_numpy_to_gpu(offsets.astype(np.uint32), stream, DataType.uint32)}
    centered = r.wrap(r.values - r.spread(r.reduce(r.values, "sum"), normalize=True))
    filler = to_storage(np.full(shape, 9.0, np.float32), dtype)
    pre = {"softmax": copy_numpy_to_gpu(filler, stream, dtype), "centered": copy_numpy_to_gpu(filler, stream, dtype)}
    plan, _ = run(ex.outputs({"softmax": r.softmax(), "centered": centered}), inputs, stream, pre)
    got_softmax = from_storage(copy_gpu_to_numpy(plan.output("softmax"), stream), dtype).astype(np.float64)
    got_centered = from_storage(copy_gpu_to_numpy(plan.output("centered"), stream), dtype).astype(np.float64)
    want_softmax, want_centered = np.full(shape, 9.0), np.full(shape, 9.0)
    for b in range(segments):
        lo, hi = offsets[b], offsets[b + 1]
        if hi > lo:
            e = np.exp(xf[lo:hi] - xf[lo:hi].max(axis=0))
            want_softmax[lo:hi] = e / e.sum(axis=0)
            want_centered[lo:hi] = xf[lo:hi] - xf[lo:hi].mean(axis=0)
    tolerance = 2e-5 if dtype == DataType.fp32 else 3e-2
    np.testing.assert_allclose(got_softmax, want_softmax, rtol=0, atol=tolerance)
    np.testing.assert_allclose(got_centered, want_centered, rtol=0, atol=tolerance * 4)


def test_dtype_and_shape_rules(stream):
    x = copy_numpy_to_gpu(np.zeros((6, 2), np.float32), stream, DataType.fp16)
    offsets = copy_numpy_to_gpu(np.array([0, 2, 6], np.uint32), stream, DataType.uint32)
    v, o = ex.input("v"), ex.input("o")
    eq = ex.compile(ex.outputs({"s": v.segment_sum(o)}), device_num=0)
    plan = eq.stamp({"v": x, "o": offsets}, stream)
    assert plan.output("s").get_data_type() == DataType.fp16 and plan.output("s").get_dimensions() == [2, 2]
    with pytest.raises(RuntimeError, match="offsets must have UINT32 or UINT64"):
        ex.compile(ex.outputs({"s": v.segment_sum(o)}), device_num=0).stamp({"v": x, "o": copy_numpy_to_gpu(np.zeros(3, np.float32), stream, DataType.fp32)}, stream)
    with pytest.raises(RuntimeError, match="output dtype to match input dtype"):
        ex.compile(ex.outputs({"s": v.segment_sum(o).with_output_dtype(DataType.fp32)}), device_num=0).stamp({"v": x, "o": offsets}, stream)
    with pytest.raises(ValueError, match="direct input"):
        v.with_ragged_runtime_extent(o + 1.0, 2, 6, 2)
    with pytest.raises(RuntimeError, match="batch size \\+ 1"):
        ex.compile(ex.outputs({"s": v.segment_sum(o, 5, 6, 2)}), device_num=0).stamp({"v": x, "o": offsets}, stream)


def staged(run_it):
    """The same expression with stage fusion off: one stage per segmented reduction, broadcast and elementwise group."""
    import os
    os.environ["THOR_DISABLE_STAGE_FUSION"] = "1"
    try:
        return run_it()
    finally:
        os.environ.pop("THOR_DISABLE_STAGE_FUSION", None)


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16], ids=lambda d: d.name)
def test_fused_and_staged_softmax_plans_agree(stream, dtype):
    """Fused: the exponentials are never stored (the sum's kernel evaluates them with the per-segment maximum read once per
    segment; the last kernel recomputes them), per-segment values are read through the row -> segment index."""
    rng = np.random.default_rng(11)
    capacity, trailing, segments = 6000, (16,), 200
    offsets = np.concatenate([[0], np.sort(rng.integers(0, 5000, segments - 1)), [5000]]).astype(np.uint32)
    x = to_storage(rng.standard_normal((capacity,) + trailing).astype(np.float32) * 2, dtype)
    r = Ragged("x", segments, capacity, trailing)
    inputs = {"x.values": copy_numpy_to_gpu(x, stream, dtype), "x.offsets": copy_numpy_to_gpu(offsets, stream, DataType.uint32)}

    def both():
        out = {}
        for name, e in (("softmax", r.softmax()), ("log_softmax", r.softmax(True))):
            filler = copy_numpy_to_gpu(to_storage(np.zeros((capacity,) + trailing, np.float32), dtype), stream, dtype)
            plan, _ = run(ex.outputs({"y": e}), inputs, stream, {"y": filler})
            out[name] = (plan.stage_kind_names(), from_storage(copy_gpu_to_numpy(plan.output("y"), stream), dtype))
        return out

    fused, reference = both(), staged(both)
    # the segment maximum and the sum of exponentials come out of one pass over the values when the arithmetic is fp32
    one_pass = ["FusedReduction", "SegmentedBroadcast", "FusedKernel"]
    assert fused["softmax"][0] == (one_pass if dtype == DataType.fp32 else ["SegmentedReduction"] + one_pass), fused["softmax"][0]
    assert reference["softmax"][0] == ["SegmentedReduction", "SegmentedBroadcast", "FusedKernel", "SegmentedReduction", "SegmentedBroadcast", "FusedKernel"]
    tolerance = 1e-6 if dtype == DataType.fp32 else 2e-3
    for name in ("softmax", "log_softmax"):
        np.testing.assert_allclose(fused[name][1], reference[name][1], rtol=0, atol=tolerance, err_msg=name)


def test_kernels_that_broadcast_other_operands_take_materialised_rows(stream):
    """A per-channel bias makes the elementwise kernel a broadcasting one: the per-segment values reach it as a stored
    [rows, E] tensor; the segmented reduction then squares the stored rows in registers."""
    rng = np.random.default_rng(5)
    capacity, e_per, segments = 700, 12, 9
    offsets = np.array([0, 50, 50, 120, 300, 301, 420, 600, 650, 700], np.uint32)
    x = rng.standard_normal((capacity, e_per)).astype(np.float32)
    bias = rng.standard_normal((1, e_per)).astype(np.float32)
    r = Ragged("x", segments, capacity, (e_per,))
    b = ex.input("bias")
    inputs = {"x.values": copy_numpy_to_gpu(x, stream, DataType.fp32), "x.offsets": copy_numpy_to_gpu(offsets, stream, DataType.uint32),
              "bias": copy_numpy_to_gpu(bias, stream, DataType.fp32)}
    centred = r.values - r.spread(r.reduce(r.values, "mean")) + b
    outputs = ex.outputs({"rows": centred, "energy": r.reduce(centred * centred, "sum")})
    plan, _ = run(outputs, inputs, stream)
    means = np.stack([x[lo:hi].mean(axis=0) if hi > lo else np.zeros(e_per) for lo, hi in zip(offsets[:-1], offsets[1:])])
    want_rows = x - np.repeat(means, np.diff(offsets), axis=0) + bias
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("rows"), stream), want_rows, rtol=1e-5, atol=1e-5)
    want_energy = np.stack([(want_rows[lo:hi] ** 2).sum(axis=0) for lo, hi in zip(offsets[:-1], offsets[1:])])
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("energy"), stream), want_energy, rtol=1e-4, atol=1e-4)
    assert plan.stage_kind_names() == ["SegmentedReduction", "SegmentedBroadcast", "FusedKernel", "FusedReduction"]


def test_segmented_reduction_of_an_expression_with_scalars_and_means(stream):
    """sum((x - mean)^2 * w) per segment with a runtime scalar: one kernel over x after the mean, nothing stored in between."""
    rng = np.random.default_rng(8)
    capacity, segments = 50000, 300
    offsets = np.concatenate([[0], np.sort(rng.integers(0, capacity, segments - 1)), [capacity]]).astype(np.uint64)
    x = rng.standard_normal((capacity, 4)).astype(np.float32)
    r = Ragged("x", segments, capacity, (4,))
    w = ex.runtime_scalar("w")
    deviation = r.values - r.spread(r.reduce(r.values, "mean"))
    outputs = ex.outputs({"scatter": r.reduce(deviation * deviation * w, "sum")})
    eq = ex.compile(outputs, device_num=0)
    plan = eq.stamp({"x.values": copy_numpy_to_gpu(x, stream, DataType.fp32), "x.offsets": copy_numpy_to_gpu(offsets, stream, DataType.uint64)}, stream)
    assert plan.stage_kind_names() == ["SegmentedReduction", "FusedReduction"]
    plan.run({"w": 0.5})
    want = np.stack([((x[lo:hi] - x[lo:hi].mean(axis=0)) ** 2).sum(axis=0) * 0.5 if hi > lo else np.zeros(4)
                     for lo, hi in zip(offsets[:-1].astype(int), offsets[1:].astype(int))])
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("scatter"), stream), want, rtol=2e-5, atol=1e-5)


# ---- backward of per-segment min / max: the segment's gradient goes to the row that won the column --------------------------------
def test_segment_min_max_backward_known_answers(stream):
    """The values and offsets of RaggedExpressionTest.cpp:1795-1824 there; winners read off by hand: min rows 1, -, 3, 5 and max
    rows 2, -, 4, 6; rows 7 and 8 belong to no segment; the empty segment's gradient goes nowhere."""
    values = np.array([1, -2, 4, 5, 7, -1, 8, 99, 100], np.float32)
    offsets = np.array([0, 3, 3, 5, 7], np.uint32)
    upstream = np.array([10, 20, 30, 40], np.float32)
    tensors = {"v": copy_numpy_to_gpu(values, stream, DataType.fp32), "o": copy_numpy_to_gpu(offsets, stream, DataType.uint32),
               "__grad_output": copy_numpy_to_gpu(upstream, stream, DataType.fp32)}
    expected = {"min": [0, 10, 0, 30, 0, 40, 0, 0, 0], "max": [0, 0, 10, 0, 30, 0, 40, 0, 0]}
    for kind in ("min", "max"):
        fwd = ex.compile(getattr(ex.input("v"), "segment_" + kind)(ex.input("o"), 4, 9, 1), device_num=0)
        plan = fwd.compile_backward(["v"], error_input_name="__grad_output").stamp(tensors, stream)
        plan.run()
        assert plan.stage_kind_names().count("SegmentedReduction") == 1 and sum("scatter_add" in d for d in plan.stage_descriptions()) == 1
        np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("v_grad"), stream), np.array(expected[kind], np.float32))


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("offsets_dtype", [DataType.uint32, DataType.uint64], ids=lambda d: d.name)
@pytest.mark.parametrize("kind", ["min", "max"])
def test_segment_min_max_backward_against_numpy(stream, kind, offsets_dtype, dtype):
    rng = np.random.default_rng(71)
    rows, width, segments = 5000, 24, 300
    cuts = np.sort(rng.integers(0, rows - 100, segments - 1))
    offsets = np.concatenate([[0], cuts, [rows - 100]])  # empty segments among them, the last 100 rows in no segment
    values = to_storage(rng.integers(-20, 21, (rows, width)).astype(np.float32) * 0.25, dtype)  # many ties: the lowest row must win
    upstream = to_storage(rng.integers(-8, 9, (segments, width)).astype(np.float32) * 0.5, dtype)
    carrier = np.uint32 if offsets_dtype == DataType.uint32 else np.uint64
    v, o = ex.input("v"), ex.input("o")
    # through elementwise work on both sides of the reduction
    loss = getattr(v * 2.0, "segment_" + kind)(o, segments, rows, width) * 3.0
    plan = ex.compile(loss, device_num=0).compile_backward(["v"], error_input_name="__grad_output").stamp(
        {"v": copy_numpy_to_gpu(values, stream, dtype), "o": copy_numpy_to_gpu(offsets.astype(carrier), stream, offsets_dtype),
         "__grad_output": copy_numpy_to_gpu(upstream, stream, dtype)}, stream)
    plan.run()
    x = from_storage(values, dtype).astype(np.float64)
    g = from_storage(upstream, dtype).astype(np.float64)
    expected = np.zeros((rows, width))
    for s in range(segments):
        lo, hi = int(offsets[s]), int(offsets[s + 1])
        if hi > lo:
            winner = lo + (np.argmin(x[lo:hi], axis=0) if kind == "min" else np.argmax(x[lo:hi], axis=0))  # first among equals
            expected[winner, np.arange(width)] = 6.0 * g[s]
    got = from_storage(copy_gpu_to_numpy(plan.output("v_grad"), stream), dtype).astype(np.float64)
    assert plan.output("v_grad").get_data_type() == dtype
    np.testing.assert_array_equal(got, expected)  # 6 * (multiples of 0.5 up to 4) is exact in bf16 too
