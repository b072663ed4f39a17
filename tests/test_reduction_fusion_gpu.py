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


def test_values_that_something_else_needs_are_still_materialised(gpu):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((32, 48)).astype(np.float32)
    ix = ex.input("x")
    sq = ix * ix
    outputs = ex.outputs({"sq": sq, "colsum": sq.reduce_sum(axis=0), "colmax": sq.reduce_max(axis=0)})
    plan, outs = run_staged(outputs, {"x": x}, DataType.fp32)
    kinds = plan.stage_kind_names()
    assert kinds == ["FusedKernel", "FusedReduction"], kinds  # sq is an output: written once, then both reductions read it together
    np.testing.assert_array_equal(outs["sq"], x * x)
    np.testing.assert_allclose(outs["colsum"].reshape(-1), (x.astype(np.float64) ** 2).sum(axis=0), rtol=1e-5)
    np.testing.assert_array_equal(outs["colmax"].reshape(-1), (x * x).max(axis=0))


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
