"""Several reductions over one geometry in a single pass, with their elementwise prologues evaluated in registers, against
the staged plan (Reduction / FusedKernel / Reduction, the reference's lowering: Utilities/Expression/EquationCompiler.cpp:7881
splitAtReductionBoundaries) and against closed forms in float64."""
from __future__ import annotations

import os

import numpy as np
import pytest

from helpers import from_storage, run_staged, to_storage
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex

pytestmark = pytest.mark.gpu


def staged(expr, inputs, dtypes, scalars=None):
    os.environ["THOR_DISABLE_ROW_FUSION"] = "1"
    try:
        return run_staged(expr, inputs, dtypes, scalars=scalars)
    finally:
        os.environ.pop("THOR_DISABLE_ROW_FUSION", None)


@pytest.mark.parametrize("dtype", [DataType.fp16, DataType.bf16, DataType.fp32], ids=lambda d: d.name)
@pytest.mark.parametrize("shape,axes", [((8, 16, 14, 14), [0, 2, 3]), ((6, 10, 33), [0]), ((5, 7, 9), [1]), ((4, 1000), [0, 1]), ((3, 100003), [1])],
                         ids=["nchw_per_channel", "columns", "middle", "all", "long_rows"])
def test_sum_and_sum_of_squares_in_one_pass(gpu, dtype, shape, axes):
    rng = np.random.default_rng(1238)
    x = to_storage(rng.standard_normal(shape).astype(np.float32), dtype)
    ix = ex.input("x")
    outputs = ex.outputs({"sum": ix.reduce_sum(axis=axes, squeeze=True), "sumsq": (ix * ix).reduce_sum(axis=axes, squeeze=True)})
    plan, outs = run_staged(outputs, {"x": x}, dtype)
    assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
    plan_s, outs_s = staged(outputs, {"x": x}, dtype)
    assert sorted(plan_s.stage_kind_names()) == ["FusedKernel", "Reduction", "Reduction"]
    xf = from_storage(x, dtype)
    sq = from_storage(to_storage(xf * xf, dtype), dtype)  # the staged plan stores x*x in the input's dtype; the fused plan rounds the same way
    want_sum = xf.astype(np.float64).sum(axis=tuple(axes))
    want_sq = sq.astype(np.float64).sum(axis=tuple(axes))
    scale = np.abs(xf).astype(np.float64).sum(axis=tuple(axes))
    for name, want, magnitude in (("sum", want_sum, scale), ("sumsq", want_sq, want_sq)):
        got = outs[name].astype(np.float64).reshape(np.shape(want))
        assert outs[name].dtype == np.float32 and outs[name].shape == outs_s[name].shape
        assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(magnitude, 1e-30)), name
        assert np.all(np.abs(got - outs_s[name].astype(np.float64).reshape(np.shape(want))) <= 2e-5 * np.maximum(magnitude, 1e-30)), name


def test_order_independent_values_match_the_staged_plan_bit_for_bit(gpu):
    rng = np.random.default_rng(4)
    x = to_storage((rng.standard_normal((12, 40, 24)) * 5).astype(np.float32), DataType.bf16)
    y = to_storage((rng.standard_normal((12, 40, 24)) * 5).astype(np.float32), DataType.bf16)
    ix, iy = ex.input("x"), ex.input("y")
    v = ix * iy + 0.5
    outputs = ex.outputs({"hi": v.reduce_max(axis=[0, 2]), "lo": v.reduce_min(axis=[0, 2]), "xmax": ix.reduce_max(axis=[0, 2])})
    plan, outs = run_staged(outputs, {"x": x, "y": y}, DataType.bf16)
    assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
    plan_s, outs_s = staged(outputs, {"x": x, "y": y}, DataType.bf16)
    assert "FusedKernel" in plan_s.stage_kind_names()
    for name in ("hi", "lo", "xmax"):
        assert outs[name].shape == (1, 40, 1)
        np.testing.assert_array_equal(outs[name], outs_s[name], err_msg=name)
    xf, yf = from_storage(x, DataType.bf16), from_storage(y, DataType.bf16)
    prod = from_storage(to_storage(xf * yf, DataType.bf16), DataType.bf16)          # bf16 multiply rounds once
    vv = from_storage(to_storage(prod + np.float32(0.5), DataType.bf16), DataType.bf16)  # then the add
    np.testing.assert_array_equal(outs["hi"].reshape(40), vv.max(axis=(0, 2)))
    np.testing.assert_array_equal(outs["lo"].reshape(40), vv.min(axis=(0, 2)))


def test_mixed_operations_scalars_and_output_dtypes(gpu):
    rng = np.random.default_rng(10)
    x = rng.uniform(0.5, 2.0, (64, 96)).astype(np.float32)
    b = np.array([0.25], dtype=np.float32)
    ix, ib, t = ex.input("x"), ex.input("b"), ex.runtime_scalar("t")
    v = (ix * t + ib)
    outputs = ex.outputs({"mean": v.reduce_mean(axis=0), "l2": v.reduce_norm2(axis=0), "l1": (ix - 1.0).reduce_norm1(axis=0),
                          "prod": ix.reduce_prod(axis=0, output_dtype=DataType.fp32), "sum16": v.reduce_sum(axis=0, output_dtype=DataType.fp16)})
    for scale in (0.5, 1.5):
        plan, outs = run_staged(outputs, {"x": x, "b": b}, DataType.fp32, scalars={"t": scale})
        assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
        v64 = x.astype(np.float64) * scale + 0.25
        np.testing.assert_allclose(outs["mean"].reshape(-1), v64.mean(axis=0), rtol=1e-5)
        np.testing.assert_allclose(outs["l2"].reshape(-1), np.sqrt((v64 ** 2).sum(axis=0)), rtol=1e-5)
        np.testing.assert_allclose(outs["l1"].reshape(-1), np.abs(x.astype(np.float64) - 1).sum(axis=0), rtol=2e-5)
        np.testing.assert_allclose(outs["prod"].reshape(-1), x.astype(np.float64).prod(axis=0), rtol=2e-5)
        assert outs["sum16"].dtype == np.float16
        np.testing.assert_allclose(outs["sum16"].reshape(-1).astype(np.float64), v64.sum(axis=0), rtol=1e-3)


def test_values_that_something_else_needs_are_written_by_the_same_pass(gpu):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((32, 48)).astype(np.float32)
    ix = ex.input("x")
    sq = ix * ix
    outputs = ex.outputs({"sq": sq, "colsum": sq.reduce_sum(axis=0), "colmax": sq.reduce_max(axis=0)})
    plan, outs = run_staged(outputs, {"x": x}, DataType.fp32)
    kinds = plan.stage_kind_names()
    assert kinds == ["FusedReduction"], kinds  # sq is an output: the pass that reduces it also writes it
    assert "elementwise_outputs=1" in plan.stage_descriptions()[0]
    np.testing.assert_array_equal(outs["sq"], x * x)
    np.testing.assert_allclose(outs["colsum"].reshape(-1), (x.astype(np.float64) ** 2).sum(axis=0), rtol=1e-5)
    np.testing.assert_array_equal(outs["colmax"].reshape(-1), (x * x).max(axis=0))
    _, outs_s = staged(outputs, {"x": x}, DataType.fp32)
    np.testing.assert_array_equal(outs["sq"], outs_s["sq"])
    np.testing.assert_array_equal(outs["colmax"], outs_s["colmax"])


@pytest.mark.parametrize("stats_of", ["input", "output"])
@pytest.mark.parametrize("shape", [(4, 16, 6, 10), (3, 8, 7, 9)], ids=lambda s: "x".join(map(str, s)))
def test_per_channel_scale_bias_relu_with_statistics_in_one_pass(gpu, shape, stats_of):
    """BASELINE config 5's three results from one read of x: y = relu(x*scale+bias) with [1,C,1,1] scale and bias, plus
    per-channel sum and sum of squares (of x, or of y)."""
    rng = np.random.default_rng(1238)
    C = shape[1]
    x = to_storage(rng.standard_normal(shape).astype(np.float32), DataType.fp16)
    scale = to_storage(rng.uniform(0.5, 1.5, (1, C, 1, 1)).astype(np.float32), DataType.fp16)
    bias = to_storage(rng.uniform(-0.1, 0.1, (1, C, 1, 1)).astype(np.float32), DataType.fp16)
    ix, isc, ib = ex.input("x"), ex.input("scale"), ex.input("bias")
    y = (ix * isc + ib).max(0.0)
    v = ix if stats_of == "input" else y
    outputs = ex.outputs({"y": y, "sum": v.reduce_sum(axis=[0, 2, 3], squeeze=True), "sumsq": (v * v).reduce_sum(axis=[0, 2, 3], squeeze=True)})
    inputs = {"x": x, "scale": scale, "bias": bias}
    plan, outs = run_staged(outputs, inputs, DataType.fp16)
    assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
    plan_s, outs_s = staged(outputs, inputs, DataType.fp16)
    assert len(plan_s.stage_kind_names()) >= 3
    # the elementwise result involves no accumulation: bit-identical to the staged plan and to fp16 arithmetic rounded per operation
    np.testing.assert_array_equal(outs["y"].view(np.uint16), outs_s["y"].view(np.uint16))
    xf, sf, bf = (from_storage(a, DataType.fp16) for a in (x, scale, bias))
    h = lambda a: from_storage(to_storage(a, DataType.fp16), DataType.fp16)
    want_y = np.maximum(h(h(xf * sf) + bf), 0)
    np.testing.assert_array_equal(from_storage(outs["y"], DataType.fp16), want_y)
    vf = xf if stats_of == "input" else want_y
    want_sum = vf.astype(np.float64).sum(axis=(0, 2, 3))
    want_sq = h(vf * vf).astype(np.float64).sum(axis=(0, 2, 3))
    assert np.all(np.abs(outs["sum"].astype(np.float64) - want_sum) <= 1e-5 * np.abs(vf).astype(np.float64).sum(axis=(0, 2, 3)) + 1e-30)
    np.testing.assert_allclose(outs["sumsq"].astype(np.float64), want_sq, rtol=1e-5)
    for name in ("sum", "sumsq"):
        np.testing.assert_allclose(outs[name], outs_s[name], rtol=2e-5, atol=1e-4)


def test_per_row_and_scalar_operands_in_row_and_column_geometries(gpu):
    rng = np.random.default_rng(15)
    x = rng.standard_normal((48, 100003)).astype(np.float32)   # rows too long for the register-resident row kernel
    w = rng.uniform(0.5, 2.0, (48, 1)).astype(np.float32)      # one weight per row: a kept operand of the row reduction
    c = np.array([0.75], dtype=np.float32)
    ix, iw, ic = ex.input("x"), ex.input("w"), ex.input("c")
    v = ix * iw + ic
    outputs = ex.outputs({"rowsum": v.reduce_sum(axis=1), "rowmax": v.reduce_max(axis=1)})
    plan, outs = run_staged(outputs, {"x": x, "w": w, "c": c}, DataType.fp32)
    assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
    v64 = x.astype(np.float64) * w + 0.75
    np.testing.assert_allclose(outs["rowsum"].reshape(-1), v64.sum(axis=1), rtol=1e-5, atol=1e-2)
    np.testing.assert_allclose(outs["rowmax"].reshape(-1), v64.max(axis=1), rtol=1e-6)
    # column geometry: one weight per column
    y = rng.standard_normal((1000, 96)).astype(np.float32)
    g = rng.uniform(0.5, 2.0, (96,)).astype(np.float32)
    iy, ig = ex.input("y"), ex.input("g")
    outputs = ex.outputs({"colsum": (iy * ig).reduce_sum(axis=0, squeeze=True), "colsq": (iy * iy).reduce_sum(axis=0, squeeze=True)})
    plan, outs = run_staged(outputs, {"y": y, "g": g}, DataType.fp32)
    assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
    np.testing.assert_allclose(outs["colsum"], (y.astype(np.float64) * g).sum(axis=0), rtol=1e-5, atol=1e-3)
    np.testing.assert_allclose(outs["colsq"], (y.astype(np.float64) ** 2).sum(axis=0), rtol=1e-5)


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16], ids=lambda d: d.name)
def test_operands_broadcast_along_some_of_the_kept_axes(gpu, dtype):
    """A [C, 1, 1] bias and a [N, 1, 1, 1] gain under [N, C, H, W] -> [N, C] (reduced over H, W): both depend on the output alone but
    have fewer elements than outputs, so their offsets are worked out of the output's number; likewise a [1, K] operand under
    [B, R, K] reduced over R (columns) and a [B, 1, 1] one there."""
    rng = np.random.default_rng(77)
    n, c, h, w = 6, 10, 9, 12
    x = to_storage(rng.standard_normal((n, c, h, w)).astype(np.float32), dtype)
    bias = to_storage(rng.standard_normal((c, 1, 1)).astype(np.float32), dtype)
    gain = to_storage(rng.uniform(0.5, 2.0, (n, 1, 1, 1)).astype(np.float32), dtype)
    ix, ib, ig = ex.input("x"), ex.input("bias"), ex.input("gain")
    v = (ix + ib) * ig
    outputs = ex.outputs({"sum": v.reduce_sum(axis=[2, 3], squeeze=True), "peak": v.reduce_max(axis=[2, 3], squeeze=True)})
    plan, outs = run_staged(outputs, {"x": x, "bias": bias, "gain": gain}, dtype)
    assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
    _, outs_s = staged(outputs, {"x": x, "bias": bias, "gain": gain}, dtype)
    xf, bf, gf = (from_storage(t, dtype).astype(np.float64) for t in (x, bias, gain))
    if dtype == DataType.fp32:
        want = (xf + bf) * gf
    else:  # 16-bit arithmetic rounds every operation
        step = from_storage(to_storage((xf + bf).astype(np.float32), dtype), dtype).astype(np.float64)
        want = from_storage(to_storage((step * gf).astype(np.float32), dtype), dtype).astype(np.float64)
    tolerance = 1e-5 if dtype == DataType.fp32 else 2e-3
    np.testing.assert_allclose(outs["sum"].reshape(n, c), want.sum(axis=(2, 3)), rtol=tolerance, atol=tolerance * 50)
    np.testing.assert_allclose(outs["peak"].reshape(n, c), want.max(axis=(2, 3)), rtol=tolerance)
    np.testing.assert_array_equal(outs["peak"], outs_s["peak"])  # order-independent: the staged plan's bits
    # columns: [B, R, K] over R with a [1, K] and a [B, 1, 1] operand
    b, r, k = 5, 700, 24
    y = rng.standard_normal((b, r, k)).astype(np.float32)
    per_k = rng.uniform(0.5, 2.0, (1, k)).astype(np.float32)
    per_b = rng.standard_normal((b, 1, 1)).astype(np.float32)
    iy, ik, ip = ex.input("y"), ex.input("per_k"), ex.input("per_b")
    outputs = ex.outputs({"a": (iy * ik + ip).reduce_sum(axis=1, squeeze=True), "b": (iy * iy).reduce_sum(axis=1, squeeze=True)})
    plan, outs = run_staged(outputs, {"y": y, "per_k": per_k, "per_b": per_b}, DataType.fp32)
    assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
    np.testing.assert_allclose(outs["a"].reshape(b, k), (y.astype(np.float64) * per_k + per_b).sum(axis=1), rtol=1e-5, atol=1e-3)
    np.testing.assert_allclose(outs["b"].reshape(b, k), (y.astype(np.float64) ** 2).sum(axis=1), rtol=1e-5)


def test_config5_per_channel_statistics_at_full_size(gpu):
    """fp16 NCHW [64, 256, 56, 56]: per-channel sum and sum of squares (fp32) in one 2-byte-per-element pass."""
    rng = np.random.default_rng(1238)
    shape = (64, 256, 56, 56)
    x = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
    ix = ex.input("x")
    outputs = ex.outputs({"sum": ix.reduce_sum(axis=[0, 2, 3], squeeze=True), "sumsq": (ix * ix).reduce_sum(axis=[0, 2, 3], squeeze=True)})
    plan, outs = run_staged(outputs, {"x": x}, DataType.fp16)
    assert plan.stage_kind_names() == ["FusedReduction"], plan.stage_descriptions()
    x64 = x.astype(np.float64)
    want_sum = x64.sum(axis=(0, 2, 3))
    sq = (x * x).astype(np.float64)  # fp16 multiply, rounded once, like the staged plan's materialised x*x
    want_sq = sq.sum(axis=(0, 2, 3))
    assert outs["sum"].shape == (256,) and outs["sumsq"].shape == (256,)
    assert np.all(np.abs(outs["sum"].astype(np.float64) - want_sum) <= 1e-5 * np.abs(x64).sum(axis=(0, 2, 3)))
    np.testing.assert_allclose(outs["sumsq"].astype(np.float64), want_sq, rtol=1e-5)
