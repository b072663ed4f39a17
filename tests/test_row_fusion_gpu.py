"""Single-pass row kernels (chains of last-axis reductions and the elementwise work between them, kept in registers)
against the staged plan of the same expression and against closed forms in float64.

The staged plan is what the reference produces for these expressions (test/Utilities/Expression/CommonInputFusionTest.cpp:281-327:
softmax lowers to Reduction, Fused, Reduction, Fused); the row kernel must give the same values up to the rounding
freedom of the fp32 accumulation order, and exactly the same values where no accumulation order is involved."""
from __future__ import annotations

import os

import numpy as np
import pytest

from helpers import from_storage, run_staged, to_storage, ulp_distance_f32
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex

pytestmark = pytest.mark.gpu


def staged(expr, inputs, dtypes, scalars=None):
    os.environ["THOR_DISABLE_ROW_FUSION"] = "1"
    try:
        return run_staged(expr, inputs, dtypes, scalars=scalars)
    finally:
        os.environ.pop("THOR_DISABLE_ROW_FUSION", None)


def softmax_expr():
    ix = ex.input("x")
    e = (ix - ix.reduce_max(axis=1)).exp()
    return e / e.reduce_sum(axis=1)


# x - rowmax promotes a 16-bit x against the fp32 maximum to fp32, so every node of the composed softmax computes in fp32 and the
# result is fp32 whatever the input's dtype: one tolerance, what 2-ulp exp, an fp32 row sum in another order and one division allow
FP32_RESULT_TOL = (1e-5, 1e-12)


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("shape", [(33, 200), (5, 2), (3, 7), (1000, 4096), (64, 4100), (9, 16384), (2, 32768), (300, 64), (4097, 8),
                                   (129, 1001), (1000, 63), (57, 4101), (300, 129), (5, 20011)],
                         ids=lambda s: "x".join(map(str, s)))
def test_softmax_single_pass_matches_staged_and_closed_form(gpu, dtype, shape):
    rng = np.random.default_rng(1237)
    x = to_storage((rng.standard_normal(shape) * 3).astype(np.float32), dtype)
    plan, outs = run_staged(softmax_expr(), {"x": x}, dtype)
    assert plan.stage_kind_names() == ["FusedRowKernel"], plan.stage_descriptions()
    if shape[1] % 4 != 0 and shape[1] >= 32:
        # rows no vector divides keep the full vector: accesses aligned to the element, the rest of the row one by one
        assert "unaligned_vectors" in plan.stage_descriptions()[0], plan.stage_descriptions()
    plan_s, outs_s = staged(softmax_expr(), {"x": x}, dtype)
    assert plan_s.stage_kind_names() == ["Reduction", "FusedKernel", "Reduction", "FusedKernel"]
    got, ref = outs["output"], outs_s["output"]
    assert got.dtype == ref.dtype and got.shape == ref.shape == shape
    xf = from_storage(x, dtype).astype(np.float64)
    p = np.exp(xf - xf.max(axis=1, keepdims=True))
    want = p / p.sum(axis=1, keepdims=True)
    assert got.dtype == np.float32
    rtol, atol = FP32_RESULT_TOL
    np.testing.assert_allclose(got.astype(np.float64), want, rtol=rtol, atol=atol)
    # against the staged plan: same values up to the order of the fp32 row sum (and, for 16-bit compute, one rounding step)
    np.testing.assert_allclose(got.astype(np.float64), ref.astype(np.float64), rtol=rtol, atol=atol)
    np.testing.assert_allclose(got.astype(np.float64).sum(axis=1), 1.0, rtol=max(rtol, 1e-5))


def test_row_longer_than_the_register_budget_uses_streaming_stages(gpu):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 70001)).astype(np.float32)
    plan, outs = run_staged(softmax_expr(), {"x": x}, DataType.fp32)
    # no register-resident row kernel; the row sum and the exp that feeds it still share one pass
    assert plan.stage_kind_names() == ["Reduction", "FusedReduction", "FusedKernel"], plan.stage_descriptions()
    x64 = x.astype(np.float64)
    p = np.exp(x64 - x64.max(axis=1, keepdims=True))
    np.testing.assert_allclose(outs["output"], p / p.sum(axis=1, keepdims=True), rtol=3e-6, atol=1e-12)


def test_rows_that_fit_only_without_kept_values_recompute_them(gpu):
    """A row of 50 257 fp32 plus its exponentials is more than a block's registers hold; the row alone fits, and the last loop
    computes the exponentials again from it."""
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((6, 50257)) * 3).astype(np.float32)
    plan, outs = run_staged(softmax_expr(), {"x": x}, DataType.fp32)
    assert plan.stage_kind_names() == ["FusedRowKernel"] and "values_recomputed" in plan.stage_descriptions()[0], plan.stage_descriptions()
    x64 = x.astype(np.float64)
    p = np.exp(x64 - x64.max(axis=1, keepdims=True))
    np.testing.assert_allclose(outs["output"], p / p.sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-12)
    _, outs_s = staged(softmax_expr(), {"x": x}, DataType.fp32)
    np.testing.assert_allclose(outs["output"], outs_s["output"], rtol=1e-5, atol=1e-12)
    # mean / variance normalisation with scale and shift: two kept values (the centred row and its square) are recomputed
    R = 28001
    xn = (rng.standard_normal((5, R)) * 2 + 0.5).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, R).astype(np.float32), rng.uniform(-1, 1, R).astype(np.float32)
    ix, ig, ib = ex.input("x"), ex.input("gamma"), ex.input("beta")
    centered = ix - ix.reduce_mean(axis=1)
    expr = centered / ((centered * centered).reduce_mean(axis=1) + 1e-5).sqrt() * ig + ib
    plan, outs = run_staged(expr, {"x": xn, "gamma": gamma, "beta": beta}, DataType.fp32)
    assert plan.stage_kind_names() == ["FusedRowKernel"] and "values_recomputed" in plan.stage_descriptions()[0], plan.stage_descriptions()
    x64 = xn.astype(np.float64)
    mu = x64.mean(axis=1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(axis=1, keepdims=True)
    np.testing.assert_allclose(outs["output"], (x64 - mu) / np.sqrt(var + 1e-5) * gamma + beta, rtol=2e-5, atol=2e-5)


def test_order_independent_parts_are_bit_identical_to_the_staged_plan(gpu):
    """x - rowmax, rowmax and rowmax - rowmin involve no accumulation order: both plans must agree bit for bit.  Division by a
    per-row value uses one reciprocal per row plus a fused correction step in the row kernel: within 1 ulp of the IEEE
    quotient of the staged plan, and equal to it almost everywhere."""
    rng = np.random.default_rng(77)
    x = to_storage(rng.standard_normal((257, 1000)).astype(np.float32) * 10, DataType.fp16)
    ix = ex.input("x")
    m = ix.reduce_max(axis=1)
    lo = ix.reduce_min(axis=1)
    outputs = ex.outputs({"centered": (ix - m) * 0.25, "rowmax": m.squeeze([1]), "range": m - lo, "scaled": (ix - m) / (m - lo + 1.0)})
    plan, outs = run_staged(outputs, {"x": x}, DataType.fp16)
    assert plan.stage_kind_names() == ["FusedRowKernel"], plan.stage_descriptions()
    _, outs_s = staged(outputs, {"x": x}, DataType.fp16)
    for name in ("centered", "rowmax", "range"):
        assert outs[name].shape == outs_s[name].shape
        np.testing.assert_array_equal(outs[name].view(np.uint8), outs_s[name].view(np.uint8), err_msg=name)
    xf = from_storage(x, DataType.fp16)
    assert outs["rowmax"].dtype == np.float32  # reductions produce fp32 unless told otherwise
    np.testing.assert_array_equal(outs["rowmax"], xf.max(axis=1))
    assert outs["scaled"].dtype == np.float32
    distance = ulp_distance_f32(outs["scaled"], outs_s["scaled"])
    assert distance.max() <= 1 and (distance != 0).mean() < 1e-3
    x64 = xf.astype(np.float64)
    exact = (x64 - x64.max(axis=1, keepdims=True)) / (x64.max(axis=1, keepdims=True) - x64.min(axis=1, keepdims=True) + 1.0)
    assert ulp_distance_f32(outs["scaled"], exact.astype(np.float32)).max() <= 2


def test_row_divisor_special_values(gpu):
    """Zeros, infinities, NaNs, huge and tiny divisors and dividends give the same results as the staged plan's IEEE division."""
    rows = np.array([[1.0, -2.0, 0.0, -0.0, np.inf, -np.inf, np.nan, 3e38, 1e-45, 1.5e-39, 7.0, 1e30],
                     [1e38, 2e38, 3e38, 1.0, 0.0, -1.0, 5.0, 6.0, 7.0, 8.0, 9.0, 10.0],
                     [1e-30, 2e-30, 1e-38, 1.0e-35, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0],
                     [0.0] * 12,
                     [np.inf, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0, 9.0, 10.0, 11.0],
                     [3.0, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0, 9.0, 10.0, 11.0]], dtype=np.float32)
    ix = ex.input("x")
    expr = ix / ix.reduce_max(axis=1) + (ix * ix) / ix.reduce_norm1(axis=1)
    plan, outs = run_staged(expr, {"x": rows}, DataType.fp32)
    assert plan.stage_kind_names() == ["FusedRowKernel"], plan.stage_descriptions()
    _, outs_s = staged(expr, {"x": rows}, DataType.fp32)
    got, ref = outs["output"], outs_s["output"]
    np.testing.assert_array_equal(np.isnan(got), np.isnan(ref))
    np.testing.assert_array_equal(np.isinf(got), np.isinf(ref))
    finite = np.isfinite(ref)
    assert ulp_distance_f32(got[finite], ref[finite]).max() <= 2


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("shape", [(8, 3, 130), (2048, 1024), (17, 4096), (8, 3, 131), (500, 1023), (77, 257)], ids=lambda s: "x".join(map(str, s)))
def test_mean_variance_normalisation_single_pass(gpu, dtype, shape):
    """y = (x - mean) / sqrt(var + eps) * gamma + beta over the last axis, gamma/beta of shape [R]."""
    rng = np.random.default_rng(99)
    R = shape[-1]
    last = len(shape) - 1
    x = to_storage((rng.standard_normal(shape) * 2 + 0.5).astype(np.float32), dtype)
    gamma = to_storage(rng.uniform(0.5, 1.5, R).astype(np.float32), dtype)
    beta = to_storage(rng.uniform(-1, 1, R).astype(np.float32), dtype)
    ix, ig, ib = ex.input("x"), ex.input("gamma"), ex.input("beta")
    mean = ix.reduce_mean(axis=last)
    centered = ix - mean
    var = (centered * centered).reduce_mean(axis=last)
    expr = centered / (var + 1e-5).sqrt() * ig + ib
    inputs = {"x": x, "gamma": gamma, "beta": beta}
    plan, outs = run_staged(expr, inputs, dtype)
    assert plan.stage_kind_names() == ["FusedRowKernel"], plan.stage_descriptions()
    _, outs_s = staged(expr, inputs, dtype)
    xf = from_storage(x, dtype).astype(np.float64)
    g, b = from_storage(gamma, dtype).astype(np.float64), from_storage(beta, dtype).astype(np.float64)
    mu = xf.mean(axis=last, keepdims=True)
    v = ((xf - mu) ** 2).mean(axis=last, keepdims=True)
    want = (xf - mu) / np.sqrt(v + 1e-5) * g + b
    rtol, atol = {DataType.fp32: (2e-5, 2e-5), DataType.fp16: (6e-3, 6e-3), DataType.bf16: (4e-2, 4e-2)}[dtype]
    got = outs["output"].astype(np.float64)
    assert got.shape == tuple(shape)
    np.testing.assert_allclose(got, want, rtol=rtol, atol=atol)
    np.testing.assert_allclose(got, outs_s["output"].astype(np.float64), rtol=rtol, atol=atol)


def test_values_needed_by_later_stages_are_written_and_everything_else_stays_on_chip(gpu):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((96, 384)).astype(np.float32)
    ix = ex.input("x")
    e = (ix - ix.reduce_max(axis=1)).exp()
    row_sum = e.reduce_sum(axis=1)               # [96, 1]
    total = row_sum.reduce_sum(axis=0)           # [1, 1]: a reduction over rows, outside the row kernel
    outputs = ex.outputs({"softmax": e / row_sum, "total": total, "lse": row_sum.ln() + ix.reduce_max(axis=1)})
    plan, outs = run_staged(outputs, {"x": x}, DataType.fp32)
    kinds = plan.stage_kind_names()
    assert kinds[0] == "FusedRowKernel" and kinds.count("FusedRowKernel") == 1 and "Reduction" in kinds[1:], kinds
    x64 = x.astype(np.float64)
    m = x64.max(axis=1, keepdims=True)
    p = np.exp(x64 - m)
    np.testing.assert_allclose(outs["softmax"], p / p.sum(axis=1, keepdims=True), rtol=3e-6)
    np.testing.assert_allclose(outs["total"].reshape(()), p.sum(), rtol=1e-5)
    np.testing.assert_allclose(outs["lse"], np.log(p.sum(axis=1, keepdims=True)) + m, rtol=1e-6)


def test_runtime_scalar_and_squeezed_results(gpu):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((40, 333)).astype(np.float32)
    ix, t = ex.input("x"), ex.runtime_scalar("t")
    scaled = ix * t
    e = (scaled - scaled.reduce_max(axis=1)).exp()
    outputs = ex.outputs({"p": e / e.reduce_sum(axis=1), "sumsq": (scaled * scaled).reduce_sum(axis=1, squeeze=True) * 0.5})
    for temperature in (0.5, 2.0):
        plan, outs = run_staged(outputs, {"x": x}, DataType.fp32, scalars={"t": temperature})
        assert plan.stage_kind_names() == ["FusedRowKernel"], plan.stage_descriptions()
        s = x.astype(np.float64) * temperature
        p = np.exp(s - s.max(axis=1, keepdims=True))
        np.testing.assert_allclose(outs["p"], p / p.sum(axis=1, keepdims=True), rtol=3e-6)
        assert outs["sumsq"].shape == (40,)
        np.testing.assert_allclose(outs["sumsq"], 0.5 * (s * s).sum(axis=1), rtol=1e-5)


def test_nan_and_inf_rows_behave_like_the_staged_plan(gpu):
    x = np.zeros((4, 96), np.float32)
    x[0, 5] = np.nan
    x[1, 7] = np.inf
    x[2, :] = -np.inf
    x[3, :] = np.linspace(-50, 50, 96)
    plan, outs = run_staged(softmax_expr(), {"x": x}, DataType.fp32)
    assert plan.stage_kind_names() == ["FusedRowKernel"]
    _, outs_s = staged(softmax_expr(), {"x": x}, DataType.fp32)
    np.testing.assert_array_equal(np.isnan(outs["output"]), np.isnan(outs_s["output"]))
    ok = ~np.isnan(outs_s["output"])
    np.testing.assert_allclose(outs["output"][ok], outs_s["output"][ok], rtol=2e-6, atol=1e-30)


# ---- Expression.softmax() / log_softmax(): the reference lowers these to a cuDNN stage (Expression.cpp:3724-3750); here they
# ---- lower to the composed form and, for [N, C] inputs, to one row kernel --------------------------------------------------
def _softmax64(x, axes, log=False):
    m = x.max(axis=axes, keepdims=True)
    p = np.exp(x - m)
    s = p.sum(axis=axes, keepdims=True)
    return (x - m) - np.log(s) if log else p / s


SOFTMAX_OUT_TOL = {DataType.fp32: 3e-6, DataType.fp16: 1.2e-3, DataType.bf16: 9e-3, DataType.fp8_e4m3: 1.2e-3}


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16, DataType.fp8_e4m3], ids=lambda d: d.name)
def test_softmax_method_on_matrices_is_one_row_kernel_and_keeps_the_input_dtype(gpu, dtype):
    rng = np.random.default_rng(31)
    x = to_storage((rng.standard_normal((65, 777)) * 2).astype(np.float32), dtype)
    xf = from_storage(x, dtype).astype(np.float64)
    out_dtype = DataType.fp16 if dtype == DataType.fp8_e4m3 else dtype  # fp8 inputs produce fp16, like the reference's softmax stage
    for build, want in ((lambda e: e.softmax(), _softmax64(xf, 1)), (lambda e: e.softmax("fast"), _softmax64(xf, 1)),
                        (lambda e: e.softmax("accurate", "instance"), _softmax64(xf, 1)), (lambda e: e.log_softmax(), _softmax64(xf, 1, log=True))):
        plan, outs = run_staged(build(ex.input("x")), {"x": x}, dtype)
        assert plan.stage_kind_names() == ["FusedRowKernel"], plan.stage_descriptions()
        assert plan.output().get_data_type() == out_dtype
        got = from_storage(outs["output"], out_dtype).astype(np.float64)
        tol = SOFTMAX_OUT_TOL[dtype]
        np.testing.assert_allclose(got, want, rtol=tol, atol=tol * 1e-2 if want.min() >= 0 else tol * 8)


def test_softmax_channel_and_instance_modes_on_nchw(gpu):
    rng = np.random.default_rng(32)
    x = rng.standard_normal((3, 6, 5, 7)).astype(np.float32)
    x64 = x.astype(np.float64)
    plan, outs = run_staged(ex.input("x").softmax(), {"x": x}, DataType.fp32)           # over C for every (n, h, w)
    assert "FusedRowKernel" not in plan.stage_kind_names()
    np.testing.assert_allclose(outs["output"], _softmax64(x64, 1), rtol=3e-6, atol=1e-9)
    plan, outs = run_staged(ex.input("x").softmax("accurate", "instance"), {"x": x}, DataType.fp32)  # over C*H*W per sample
    np.testing.assert_allclose(outs["output"], _softmax64(x64, (1, 2, 3)), rtol=3e-6, atol=1e-9)
    plan, outs = run_staged(ex.input("x").log_softmax("instance"), {"x": x}, DataType.fp32)
    np.testing.assert_allclose(outs["output"], _softmax64(x64, (1, 2, 3), log=True), rtol=3e-6, atol=3e-6)
    with pytest.raises(RuntimeError, match="axis"):
        run_staged(ex.input("x").softmax(), {"x": x.reshape(-1)}, DataType.fp32)
