"""GPU parity of the Expression compiler (fused elementwise / broadcast kernels, staged reductions) against closed forms.

The oracle for elementwise work is the mathematics itself: float64 closed forms bounded in ulps for fp32, and exact
per-operation rounding for fp16 / bf16 arithmetic (numpy float16 arithmetic rounds every operation; bf16 is modelled as fp32
arithmetic followed by one RNE rounding, which is exact because 24 >= 2*8+2).  Tolerances are the reference's own where
it only pins a tolerance (bindings/python/test/core/physical/test_expression_numerical.py:24-38)."""
import os

import numpy as np
import pytest
import scipy.special as sp

import oracle
from helpers import (FLOAT_DTYPES, copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, gpu_tensor, rtol_atol, run_expr, run_staged, to_storage,
                     ulp_distance_f32)
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex

pytestmark = pytest.mark.gpu


def rnd(x, dtype):
    """fp32 values rounded through `dtype` storage."""
    return from_storage(to_storage(np.asarray(x, dtype=np.float32), dtype), dtype)


def sigmoid64(x):
    x = x.astype(np.float64)
    return np.exp(-np.maximum(-x, 0)) / (1 + np.exp(-np.abs(x)))


# ---- BASELINE config 1 ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 1 << 20, (1 << 20) + 1])
def test_config1_fused_elementwise(gpu, n):
    """out = (a*b + c) * sigmoid(d), four fp32 inputs ~ U(-1,1), seed 1234."""
    rng = np.random.default_rng(1234)
    a, b, c, d = (rng.uniform(-1, 1, n).astype(np.float32) for _ in range(4))
    ea, eb, ec, ed = (ex.input(k) for k in "abcd")
    expr = (ea * eb + ec) * ed.sigmoid()
    plan, outs = run_staged(expr, {"a": a, "b": b, "c": c, "d": d}, DataType.fp32)
    assert plan.stage_kind_names() == ["FusedKernel"]
    got = outs["output"]
    a64, b64, c64 = a.astype(np.float64), b.astype(np.float64), c.astype(np.float64)
    exact = (a64 * b64 + c64) * sigmoid64(d)
    # sigmoid within 2 ulp, one rounding each for a*b+c (fused or not) and the final product: 4 ulp of the result, plus
    # the rounding of the cancelling sum a*b+c (one ulp of its larger term) carried through the product
    sig = sigmoid64(d)
    bound = 4 * np.spacing(np.abs(exact).astype(np.float32)).astype(np.float64) + np.spacing(np.maximum(np.abs(a64 * b64), np.abs(c64)).astype(np.float32)) * sig
    assert np.all(np.abs(got.astype(np.float64) - exact) <= bound)
    np.testing.assert_allclose(got, exact, rtol=3e-5, atol=3e-6)
    if n >= 4:
        assert "flat(vec=4)" in plan.stage_descriptions()[0]


def test_sigmoid_structure_and_extremes(gpu):
    """The stable form stays finite at +-1000 (bindings/python/test/core/physical/test_expression_stable_activations.py:168-191)."""
    x = np.array([-1000, -100, -20, -1, -1e-8, 0, 1e-8, 1, 20, 100, 1000], dtype=np.float32)
    got = run_expr(ex.input("x").sigmoid(), {"x": x}, DataType.fp32)
    assert np.all(np.isfinite(got))
    assert np.all(ulp_distance_f32(got, sigmoid64(x).astype(np.float32)) <= 2)
    assert got[0] == 0.0 and got[-1] == 1.0 and got[5] == 0.5
    sp_got = run_expr(ex.input("x").softplus(), {"x": x}, DataType.fp32)
    want = np.maximum(x.astype(np.float64), 0) + np.log1p(np.exp(-np.abs(x.astype(np.float64))))
    assert np.all(ulp_distance_f32(sp_got, want.astype(np.float32)) <= 2)


# ---- fp32 unary functions within ulps of the float64 closed form ---------------------------------------------------------------
UNARY = [
    ("exp", np.exp, (-20, 20), 2), ("exp2", np.exp2, (-30, 30), 2), ("expm1", np.expm1, (-5, 5), 2), ("exp10", lambda v: 10.0 ** v, (-8, 8), 2),
    ("ln", np.log, (1e-6, 1e6), 2), ("log1p", np.log1p, (-0.9, 100), 2), ("log2", np.log2, (1e-6, 1e6), 2), ("log10", np.log10, (1e-6, 1e6), 2),
    ("sqrt", np.sqrt, (0, 1e6), 0), ("tanh", np.tanh, (-10, 10), 2), ("sin", np.sin, (-6.5, 6.5), 2), ("cos", np.cos, (-6.5, 6.5), 2),
    ("tan", np.tan, (-1.5, 1.5), 3), ("asin", np.arcsin, (-1, 1), 3), ("acos", np.arccos, (-1, 1), 2), ("atan", np.arctan, (-50, 50), 2),
    ("sinh", np.sinh, (-10, 10), 3), ("cosh", np.cosh, (-10, 10), 2), ("asinh", np.arcsinh, (-100, 100), 3), ("acosh", np.arccosh, (1, 100), 3),
    ("atanh", np.arctanh, (-0.99, 0.99), 3), ("erf", sp.erf, (-4, 4), 2), ("erfc", sp.erfc, (-3, 8), 4), ("erfcx", sp.erfcx, (-3, 50), 4),
    ("erfinv", sp.erfinv, (-0.999, 0.999), 3), ("erfcinv", sp.erfcinv, (0.001, 1.999), 6), ("tgamma", sp.gamma, (0.1, 30), 8),
    ("lgamma", sp.gammaln, (3.0, 1000), 4), ("digamma", sp.digamma, (2.0, 100), 16), ("normcdf", sp.ndtr, (-8, 8), 8),
    ("abs", np.abs, (-10, 10), 0), ("ceil", np.ceil, (-10, 10), 0), ("floor", np.floor, (-10, 10), 0), ("trunc", np.trunc, (-10, 10), 0),
    ("sigmoid", sigmoid64, (-30, 30), 2), ("gelu", lambda v: v * sp.ndtr(v), (-6, 6), 8), ("swish", lambda v: v * sigmoid64(v), (-30, 30), 3),
    ("relu6", lambda v: np.minimum(np.maximum(v, 0), 6), (-10, 10), 0), ("selu", None, (-5, 5), 3), ("mish", None, (-10, 10), 4),
]


@pytest.mark.parametrize("name,ref,domain,max_ulp", UNARY, ids=[u[0] for u in UNARY])
def test_fp32_unary_within_ulps(gpu, name, ref, domain, max_ulp):
    rng = np.random.default_rng(11)
    x = rng.uniform(domain[0], domain[1], 20011).astype(np.float32)
    got = run_expr(getattr(ex.input("x"), name)(), {"x": x}, DataType.fp32)
    x64 = x.astype(np.float64)
    if name == "selu":
        want = 1.05070098 * np.maximum(x64, 0) + 1.758099326 * np.expm1(np.minimum(x64, 0))
    elif name == "mish":
        want = x64 * np.tanh(np.maximum(x64, 0) + np.log1p(np.exp(-np.abs(x64))))
    else:
        want = ref(x64)
    worst = ulp_distance_f32(got, want.astype(np.float32)).max()
    assert worst <= max_ulp, f"{name}: {worst} ulp"


def test_round_is_half_away_from_zero_and_minmax_ignore_nan(gpu):
    x = np.array([-2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 2.4999], dtype=np.float32)
    assert run_expr(ex.input("x").round(), {"x": x}, DataType.fp32).tolist() == [-3, -2, -1, 1, 2, 3, 2]
    a = np.array([1.0, np.nan, 3.0, np.nan], dtype=np.float32)
    b = np.array([2.0, 5.0, np.nan, np.nan], dtype=np.float32)
    mx = run_expr(ex.input("a").max(ex.input("b")), {"a": a, "b": b}, DataType.fp32)
    mn = run_expr(ex.input("a").min(ex.input("b")), {"a": a, "b": b}, DataType.fp32)
    assert mx[:3].tolist() == [2.0, 5.0, 3.0] and np.isnan(mx[3])  # fmaxf semantics: the number wins
    assert mn[:3].tolist() == [1.0, 5.0, 3.0] and np.isnan(mn[3])


# ---- arithmetic in every float dtype ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", FLOAT_DTYPES, ids=lambda d: d.name)
def test_add_sub_mul_div_numerical(gpu, dtype):
    """((x + y) - 2) * (x / (y + 1)), the reference's test_add_sub_mul_div_numerical."""
    x_np = to_storage(np.array([1, 2, 3, 4, 5, 6], dtype=np.float32), dtype)
    y_np = to_storage(np.array([2, 3, 4, 5, 6, 7], dtype=np.float32), dtype)
    x, y = ex.input("x"), ex.input("y")
    got = from_storage(run_expr(((x + y) - 2.0) * (x / (y + 1.0)), {"x": x_np, "y": y_np}, dtype), dtype)
    compute = DataType.fp16 if dtype in (DataType.fp8_e4m3, DataType.fp8_e5m2) else dtype
    xf, yf = from_storage(x_np, dtype), from_storage(y_np, dtype)
    s = rnd(xf + yf, compute)
    m = rnd(s - 2.0, compute)
    den = rnd(yf + 1.0, compute)
    q = rnd(xf / den, compute)
    want = rnd(rnd(m * q, compute), dtype)
    rtol, atol = rtol_atol(dtype)
    np.testing.assert_allclose(got, want, rtol=rtol, atol=atol)
    if dtype in (DataType.fp16, DataType.bf16, DataType.fp32):
        np.testing.assert_array_equal(got, want)  # every operation is correctly rounded: bit-exact


@pytest.mark.parametrize("dtype", [DataType.fp16, DataType.bf16], ids=lambda d: d.name)
def test_16bit_arithmetic_rounds_after_every_operation_bit_exact(gpu, dtype):
    rng = np.random.default_rng(21)
    n = 100003
    a, b, c = (to_storage(rng.standard_normal(n).astype(np.float32), dtype) for _ in range(3))
    af, bf, cf = (from_storage(v, dtype) for v in (a, b, c))
    x, y, z = ex.input("a"), ex.input("b"), ex.input("c")
    got = from_storage(run_expr((x * y + z).max(0.0) - y, {"a": a, "b": b, "c": c}, dtype), dtype)
    want = rnd(np.maximum(rnd(rnd(af * bf, dtype) + cf, dtype), 0) - bf, dtype)
    np.testing.assert_array_equal(got, want)


def test_mixed_dtypes_promote_like_the_reference(gpu):
    """fp16 (+) bf16 -> fp32, anything (+) fp32 -> fp32, fp8 computes in fp16 (ExpressionDTypeResolution.cpp:277-307)."""
    stream = ph.Stream(0)
    h = to_storage(np.array([1.5, 2.25, -3.0, 1000.0], np.float32), DataType.fp16)
    b = to_storage(np.array([0.1, 0.2, 0.3, 0.4], np.float32), DataType.bf16)
    eq = ex.compile(ex.input("h") * ex.input("b"), 0)
    inputs = {"h": copy_numpy_to_gpu(h, stream, DataType.fp16), "b": copy_numpy_to_gpu(b, stream, DataType.bf16)}
    dims, out_dtype = eq.get_output_shape(inputs)
    assert out_dtype == DataType.fp32 and dims == [4]
    plan = eq.stamp(inputs, stream)
    plan.run()
    got = copy_gpu_to_numpy(plan.output(), stream)
    np.testing.assert_array_equal(got, from_storage(h, DataType.fp16) * from_storage(b, DataType.bf16))
    e4 = to_storage(np.array([0.5, 1.5, -2.0, 3.0], np.float32), DataType.fp8_e4m3)
    eq = ex.compile(ex.input("x") + ex.input("x"), 0)
    inputs = {"x": copy_numpy_to_gpu(e4, stream, DataType.fp8_e4m3)}
    assert eq.get_output_shape(inputs)[1] == DataType.fp8_e4m3
    plan = eq.stamp(inputs, stream)
    plan.run()
    np.testing.assert_array_equal(from_storage(copy_gpu_to_numpy(plan.output(), stream), DataType.fp8_e4m3), [1.0, 3.0, -4.0, 6.0])


def test_compare_where_logic_and_casts(gpu):
    x = np.array([-2.0, -0.5, 0.0, 0.5, 2.0, np.nan], dtype=np.float32)
    y = np.array([1.0, -0.5, 1.0, 0.25, 3.0, 0.0], dtype=np.float32)
    ix, iy = ex.input("x"), ex.input("y")
    assert run_expr(ex.where(ix > iy, ix, iy), {"x": x, "y": y}, DataType.fp32)[:5].tolist() == [1.0, -0.5, 1.0, 0.5, 3.0]
    got = run_expr((ix <= iy).logical_and(ix != 0.0), {"x": x, "y": y}, DataType.fp32, out_dtype=DataType.boolean)
    assert got.tolist() == [1, 1, 0, 0, 1, 0]
    assert run_expr(ix.threshold(0.0, -7.0), {"x": x}, DataType.fp32)[:5].tolist() == [-7.0, -7.0, -7.0, 0.5, 2.0]
    assert run_expr(ix.cast(DataType.int32), {"x": x[:5] * 3}, DataType.fp32, out_dtype=DataType.int32).tolist() == [-6, -1, 0, 1, 6]
    assert from_storage(run_expr(ix.cast(DataType.bf16), {"x": y * 1.001}, DataType.fp32, out_dtype=DataType.bf16), DataType.bf16).tolist() == \
        rnd(y * np.float32(1.001), DataType.bf16).tolist()
    ints = np.array([1, -2, 300, 7], dtype=np.int32)
    # integer tensors enter float arithmetic through an explicit cast (the value dtype of an input defaults to its tensor's)
    got = run_expr(ex.input("i").cast(DataType.fp32) * 0.5, {"i": ints}, DataType.int32, out_dtype=DataType.fp32)
    assert got.tolist() == [0.5, -1.0, 150.0, 3.5]
    got = run_expr(ex.input("i", output_dtype=DataType.fp32) * 0.5, {"i": ints}, DataType.int32, out_dtype=DataType.fp32)
    assert got.tolist() == [0.5, -1.0, 150.0, 3.5]
    # 64-bit integers of every magnitude, either side of the ties of a 24-bit significand: the cast rounds once, to nearest even
    # (generated code converts through 32-bit halves: the compiler's expansion of the cast would shift 64 bits by a register amount)
    ties = [(1 << e) + (1 << (e - 24)) + d for e in range(24, 63) for d in (-1, 0, 1)] + [(1 << e) + 3 * (1 << (e - 24)) for e in range(24, 62)]
    for carrier, dtype, values in ((np.int64, DataType.int64, [0, 1, -1, -(1 << 63), (1 << 63) - 1] + ties + [-t for t in ties]),
                                   (np.uint64, DataType.uint64, [0, 1, (1 << 64) - 1, (1 << 63) + (1 << 39)] + ties)):
        wide = np.array(values, dtype=carrier)
        got = run_expr(ex.input("i").cast(DataType.fp32) * 1.0, {"i": wide}, dtype, out_dtype=DataType.fp32)
        np.testing.assert_array_equal(got.view(np.uint32), wide.astype(np.float32).view(np.uint32))


def test_constants_fold_and_identities_vanish(gpu):
    x = np.linspace(-2, 2, 37, dtype=np.float32)
    ix = ex.input("x")
    plan, outs = run_staged((ix + 0.0) * 1.0 + (ex.constant_scalar(2.0) * 3.0 - 1.0) / 5.0, {"x": x}, DataType.fp32)
    np.testing.assert_array_equal(outs["output"], x + np.float32(1.0))
    src = plan.stage_source(0)
    body = src[src.index("fused_kernel"):]
    assert "1.0f" in body and "3.0f" not in body and "5.0f" not in body  # (2*3-1)/5 was folded to 1 on the host


def test_runtime_scalars(gpu):
    x = np.arange(8, dtype=np.float32)
    expr = ex.input("x") * ex.runtime_scalar("alpha") + ex.runtime_scalar("beta")
    got = run_expr(expr, {"x": x}, DataType.fp32, scalars={"alpha": 2.5, "beta": -1.0})
    np.testing.assert_array_equal(got, x * np.float32(2.5) - 1)
    with pytest.raises(RuntimeError, match="alpha|beta"):
        run_expr(expr, {"x": x}, DataType.fp32, scalars={"alpha": 2.5})


# ---- broadcasting ------------------------------------------------------------------------------------------------------------------
def test_config5_shaped_per_channel_broadcast_fp16_bit_exact(gpu):
    """y = relu(x * scale + bias) on NCHW fp16 with [1,C,1,1] scale and bias; every op rounds to fp16 (no FMA)."""
    rng = np.random.default_rng(1238)
    N, C, H, W = 4, 16, 14, 14
    x = to_storage(rng.standard_normal((N, C, H, W)).astype(np.float32), DataType.fp16)
    scale = to_storage(rng.uniform(0.5, 1.5, (1, C, 1, 1)).astype(np.float32), DataType.fp16)
    bias = to_storage(rng.uniform(-0.1, 0.1, (1, C, 1, 1)).astype(np.float32), DataType.fp16)
    expr = (ex.input("x") * ex.input("scale") + ex.input("bias")).max(0.0)
    plan, outs = run_staged(expr, {"x": x, "scale": scale, "bias": bias}, DataType.fp16)
    want = np.maximum((x * scale).astype(np.float16) + bias, np.float16(0)).astype(np.float16)
    np.testing.assert_array_equal(outs["output"].view(np.uint16), want.view(np.uint16))
    assert plan.stage_kind_names() == ["FusedKernel"]
    assert "broadcast(" in plan.stage_descriptions()[0] and "vec=4" in plan.stage_descriptions()[0]


BROADCASTS = [
    ((4, 5), (5,)), ((4, 5), (4, 1)), ((4, 1), (1, 5)), ((2, 3, 4), (3, 1)), ((2, 3, 4), (1, 1, 4)), ((6, 1, 8), (1, 7, 1)), ((3, 4, 5, 6), (4, 1, 6)),
    ((1,), (3, 2)), ((2, 3, 64), (64,)), ((2, 3, 64), (2, 1, 64)), ((16, 128), (16, 1)), ((5, 7, 9), (5, 7, 9)),
]


@pytest.mark.parametrize("sa,sb", BROADCASTS, ids=lambda s: str(s))
@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.bf16], ids=lambda d: d.name)
def test_numpy_broadcasting_semantics(gpu, sa, sb, dtype):
    rng = np.random.default_rng(5)
    a = to_storage(rng.standard_normal(sa).astype(np.float32), dtype)
    b = to_storage(rng.standard_normal(sb).astype(np.float32), dtype)
    plan, outs = run_staged(ex.input("a") * ex.input("b") - ex.input("a"), {"a": a, "b": b}, dtype)
    af, bf = from_storage(a, dtype), from_storage(b, dtype)
    want = rnd(rnd(af * bf, dtype) - af, dtype)
    got = from_storage(outs["output"], dtype)
    assert got.shape == np.broadcast_shapes(sa, sb)
    if dtype == DataType.fp32:
        # fp32 stages may contract a*b-a into one fused multiply-add, as the reference's -fmad=true does
        fused = (af.astype(np.float64) * bf.astype(np.float64) - af.astype(np.float64)).astype(np.float32)
        assert np.all((got == want) | (got == fused))
    else:
        np.testing.assert_array_equal(got, want)


ODD_BROADCASTS = [
    ((129, 1001), (1001,), (129, 1)), ((7, 33, 125), (33, 1), (125,)), ((3, 1367), (1, 1367), (3, 1)), ((4099, 3), (3,), (4099, 1)),
    ((5, 1, 821), (1, 9, 821), (9, 1)), ((64, 65), (64, 65), (65,)),
]


@pytest.mark.parametrize("sa,sb,sc", ODD_BROADCASTS, ids=lambda s: str(s))
@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
def test_broadcasts_whose_innermost_extent_no_vector_divides(gpu, sa, sb, sc, dtype):
    """Rows of 1001, 125, 3 ... elements: lanes own vectors of the dense output that straddle rows, and the broadcast operands are
    read at coordinates carried along the vector.  Same results as the element-by-element form, bit for bit in 16-bit arithmetic."""
    rng = np.random.default_rng(11)
    a, b, c = (to_storage(rng.standard_normal(shape).astype(np.float32), dtype) for shape in (sa, sb, sc))
    plan, outs = run_staged((ex.input("a") + ex.input("b")) * ex.input("c"), {"a": a, "b": b, "c": c}, dtype)
    af, bf, cf = (from_storage(v, dtype) for v in (a, b, c))
    want = rnd(rnd(af + bf, dtype) * cf, dtype)
    got = from_storage(outs["output"], dtype)
    assert got.shape == want.shape
    np.testing.assert_array_equal(got, want)
    if want.size >= 4096:
        assert "vectors_straddle_rows" in plan.stage_descriptions()[0], plan.stage_descriptions()


def test_strided_view_inputs(gpu):
    stream = ph.Stream(0)
    x = np.arange(30, dtype=np.float32).reshape(5, 6)
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    tr = t.alias_view([6, 5], [1, 6])
    eq = ex.compile(ex.input("x") * 2.0 + ex.input("y"), 0)
    y = copy_numpy_to_gpu(np.ones((6, 5), np.float32), stream, DataType.fp32)
    plan = eq.stamp({"x": tr, "y": y}, stream)
    plan.run()
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output(), stream), x.T * 2 + 1)


def test_multiple_outputs_share_one_kernel(gpu):
    x = np.linspace(-3, 3, 1001, dtype=np.float32)
    y = np.linspace(1, 2, 1001, dtype=np.float32)
    ix, iy = ex.input("x"), ex.input("y")
    outputs = ex.outputs({"sum": ix + iy, "prod": ix * iy, "third": (ix + iy) * (ix * iy)})
    plan, outs = run_staged(outputs, {"x": x, "y": y}, DataType.fp32)
    np.testing.assert_array_equal(outs["sum"], x + y)
    np.testing.assert_array_equal(outs["prod"], x * y)
    np.testing.assert_array_equal(outs["third"], (x + y) * (x * y))
    kinds = plan.stage_kind_names()
    assert kinds.count("FusedKernel") == len(kinds) and len(kinds) <= 2


# ---- staged reductions ----------------------------------------------------------------------------------------------------------------
@pytest.fixture
def staged_only():
    os.environ["THOR_DISABLE_ROW_FUSION"] = "1"
    yield
    os.environ.pop("THOR_DISABLE_ROW_FUSION", None)


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
def test_reduce_sum_with_prologue_and_epilogue(gpu, staged_only, dtype):
    rng = np.random.default_rng(2)
    x = to_storage(rng.uniform(0.5, 2.0, (6, 37)).astype(np.float32), dtype)
    ix = ex.input("x")
    expr = ((ix * ix).reduce_sum(axis=1, squeeze=False) + 1.0).sqrt()
    plan, outs = run_staged(expr, {"x": x}, dtype)
    assert plan.stage_kind_names() == ["FusedKernel", "Reduction", "FusedKernel"]
    xf = from_storage(x, dtype)
    sq = rnd(xf * xf, dtype)  # the producer materialises in its own storage dtype
    want = np.sqrt(sq.astype(np.float64).sum(axis=1, keepdims=True) + 1.0)
    got = outs["output"]
    assert got.dtype == np.float32 and got.shape == (6, 1)
    np.testing.assert_allclose(got, want, rtol=1e-5)


def test_squeeze_semantics_and_output_dtypes(gpu, staged_only):
    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    ix = ex.input("x")
    for kwargs, shape in [({"axis": 1, "squeeze": False}, (2, 1, 4)), ({"axis": 1, "squeeze": True}, (2, 4)), ({"axis": [0, 2], "squeeze": [0]}, (3, 1)),
                          ({"axis": None, "squeeze": False}, (1, 1, 1)), ({"axis": None, "squeeze": True}, (1,)), ({"axis": [1, 2], "squeeze": 2}, (2, 1))]:
        _, outs = run_staged(ix.reduce_sum(**kwargs), {"x": x}, DataType.fp32)
        axes = kwargs["axis"] if kwargs["axis"] is not None else (0, 1, 2)
        want = x.sum(axis=tuple(axes) if not isinstance(axes, int) else axes, keepdims=True).reshape(shape)
        assert outs["output"].shape == shape
        np.testing.assert_array_equal(outs["output"], want)
    for od in (DataType.fp16, DataType.bf16, DataType.fp32):
        _, outs = run_staged(ix.reduce_sum(axis=1, squeeze=True, output_dtype=od), {"x": x * 1.25}, DataType.fp32)
        np.testing.assert_array_equal(from_storage(outs["output"], od), rnd((x * 1.25).sum(axis=1), od))
    _, outs = run_staged(ix.reduce_mean(axis=[0, 2], squeeze=True) * 2.0, {"x": x}, DataType.fp32)
    np.testing.assert_allclose(outs["output"], x.mean(axis=(0, 2)) * 2, rtol=1e-6)


def test_argmin_argmax_staged(gpu, staged_only):
    x = np.array([[1.0, 1.0, 3.0, 1.0], [np.nan, 0.0, np.nan, -4.0]], dtype=np.float32)
    _, outs = run_staged(ex.input("x").argmin(axis=1, squeeze=True), {"x": x}, DataType.fp32)
    assert outs["output"].dtype == np.uint32 and outs["output"].tolist() == [0, 0]
    y = np.array([[5.0, 5.0, 3.0, 5.0], [-1.0, np.nan, np.nan, 8.0]], dtype=np.float32)
    plan, outs = run_staged(ex.input("x").argmax(axis=1, squeeze=True), {"x": y}, DataType.fp32)
    assert outs["output"].tolist() == [0, 1] and plan.stage_kind_names() == ["ArgMinMax"]
    z = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    z[1, 2, 1] = 100
    _, outs = run_staged(ex.input("x").argmax(axis=[1, 2], squeeze=False), {"x": z}, DataType.fp32)
    assert outs["output"].shape == (2, 1, 1) and outs["output"].reshape(-1).tolist() == [11, 9]


def test_composed_softmax_staged_matches_reference_plan_shape(gpu, staged_only):
    """exp(x - rowmax) / rowsum splits into Reduction, Fused, Reduction, Fused (CommonInputFusionTest.cpp:281-327)."""
    rng = np.random.default_rng(1237)
    x = to_storage((rng.standard_normal((33, 200)) * 3).astype(np.float32), DataType.bf16)
    ix = ex.input("x")
    e = (ix - ix.reduce_max(axis=1)).exp()
    expr = e / e.reduce_sum(axis=1)
    plan, outs = run_staged(expr, {"x": x}, DataType.bf16)
    assert plan.stage_kind_names() == ["Reduction", "FusedKernel", "Reduction", "FusedKernel"]
    xf = from_storage(x, DataType.bf16).astype(np.float64)
    p = np.exp(xf - xf.max(axis=1, keepdims=True))
    want = p / p.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(outs["output"], want, rtol=2e-2, atol=2e-3)
    np.testing.assert_allclose(outs["output"].astype(np.float64).sum(axis=1), 1.0, rtol=2e-2)


def test_preallocated_outputs_and_errors(gpu, staged_only):
    stream = ph.Stream(0)
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    eq = ex.compile(ex.input("x").reduce_min(axis=1, squeeze=True), 0)
    tx = copy_numpy_to_gpu(x, stream, DataType.fp32)
    out = gpu_tensor([3], DataType.fp32)
    plan = eq.stamp({"x": tx}, stream, preallocated_outputs={"output": out})
    plan.run()
    assert plan.output().mem_ptr() == out.mem_ptr()
    np.testing.assert_array_equal(copy_gpu_to_numpy(out, stream), x.min(axis=1))
    with pytest.raises(RuntimeError, match="shape"):
        eq.stamp({"x": tx}, stream, preallocated_outputs={"output": gpu_tensor([4], DataType.fp32)})
    with pytest.raises(RuntimeError, match="dtype"):
        eq.stamp({"x": tx}, stream, preallocated_outputs={"output": gpu_tensor([3], DataType.fp16)})
    with pytest.raises(RuntimeError, match="Missing required input"):
        eq.stamp({}, stream)
    with pytest.raises(RuntimeError, match="reduction stage"):
        eq.run({"x": tx}, out, stream)  # the convenience run is for fused-kernel-only plans
    with pytest.raises(RuntimeError, match="broadcast"):
        run_staged(ex.input("a") + ex.input("b"), {"a": np.zeros((3, 4), np.float32), "b": np.zeros((5,), np.float32)}, DataType.fp32)


def test_kernels_are_cached_across_stamps_and_sizes(gpu):
    stream = ph.Stream(0)
    eq = ex.compile(ex.input("p") * 3.0 - ex.input("q").exp(), 0)
    before = ph.compiled_kernel_count()
    for n in (1024, 4096, 1 << 16):
        a = copy_numpy_to_gpu(np.ones(n, np.float32), stream, DataType.fp32)
        b = copy_numpy_to_gpu(np.zeros(n, np.float32), stream, DataType.fp32)
        plan = eq.stamp({"p": a, "q": b}, stream)
        plan.run()
        assert np.all(copy_gpu_to_numpy(plan.output(), stream) == 2.0)
    assert ph.compiled_kernel_count() - before <= 1  # one flat kernel serves every size
    eq2 = ex.compile(ex.input("p") * 3.0 - ex.input("q").exp(), 0)  # an equal expression built again hits the global cache
    a = copy_numpy_to_gpu(np.ones(8, np.float32), stream, DataType.fp32)
    eq2.stamp({"p": a, "q": a}, stream).run()
    assert ph.compiled_kernel_count() - before <= 1


# ---- conditional outputs (Outputs::ifElse / ifElifElse): the reference's cases, test_expression_outputs.py:625-760 there ---------------
@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def _scalar(value, stream):
    return copy_numpy_to_gpu(np.array([value], np.float32), stream, DataType.fp32)


def test_if_elif_else_takes_the_first_matching_branch(stream):
    x, selector = ex.input("x"), ex.input("selector")
    conditional = ex.if_elif_else(selector > 2.0, ex.outputs({"y": x * 10.0}),
                                  [(selector > 1.0, ex.outputs({"y": x * 20.0})), (selector > 0.0, ex.outputs({"y": x * 30.0}))],
                                  ex.outputs({"y": x * 40.0}))
    equation = conditional.compile(device_num=0)
    x_gpu = copy_numpy_to_gpu(np.array([1.0, 2.0], np.float32), stream, DataType.fp32)
    selector_gpu = _scalar(0.0, stream)
    plan = equation.stamp({"x": x_gpu, "selector": selector_gpu}, stream)
    assert plan.stage_kind_names() == ["FusedKernel"]  # every branch and the selection in one kernel
    for value, expected in [(3.0, [10.0, 20.0]), (2.0, [20.0, 40.0]), (1.0, [30.0, 60.0]), (-1.0, [40.0, 80.0])]:
        selector_gpu.copy_from_async(_scalar(value, stream), stream)  # the predicate is read on the device at every run
        plan.run()
        np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("y"), stream), np.array(expected, np.float32))


def test_if_else_with_a_device_predicate_several_outputs_and_a_poisoned_branch(stream):
    """Values of the branch that is not taken never reach an output, NaN and infinity included; reductions and several outputs
    are allowed inside the branches."""
    x = ex.input("x")
    predicate = ex.input("predicate_value") > 0.0
    conditional = ex.if_else(predicate, ex.outputs({"y": x + 10.0, "total": x.reduce_sum(axis=0)}),
                             ex.outputs({"y": (x - x) / (x - x), "total": x.reduce_max(axis=0) * float("inf")}))
    equation = conditional.compile(device_num=0)
    x_gpu = copy_numpy_to_gpu(np.array([1.0, 2.0, 3.0, 4.0], np.float32), stream, DataType.fp32)
    taken = equation.stamp({"x": x_gpu, "predicate_value": _scalar(1.0, stream)}, stream)
    taken.run()
    np.testing.assert_array_equal(copy_gpu_to_numpy(taken.output("y"), stream), np.array([11.0, 12.0, 13.0, 14.0], np.float32))
    np.testing.assert_array_equal(copy_gpu_to_numpy(taken.output("total"), stream).reshape(-1), np.array([10.0], np.float32))
    other = equation.stamp({"x": x_gpu, "predicate_value": _scalar(-1.0, stream)}, stream)
    other.run()
    assert np.all(np.isnan(copy_gpu_to_numpy(other.output("y"), stream)))
    assert np.all(np.isinf(copy_gpu_to_numpy(other.output("total"), stream)))


def test_the_gradient_of_a_conditional_flows_into_the_branch_that_was_taken(stream):
    x, predicate_value = ex.input("x"), ex.input("predicate_value")
    conditional = ex.if_else(predicate_value > 0.0, ex.outputs({"y": x * x}), ex.outputs({"y": x * 3.0}))
    backward = conditional.compile(device_num=0).compile_backward(["x"], error_input_name="dy")
    x_gpu = copy_numpy_to_gpu(np.array([-2.0, -1.0, 2.0, 4.0], np.float32), stream, DataType.fp32)
    dy_gpu = copy_numpy_to_gpu(np.array([1.0, 2.0, 3.0, 4.0], np.float32), stream, DataType.fp32)
    for value, expected in [(1.0, [-4.0, -4.0, 12.0, 32.0]), (-1.0, [3.0, 6.0, 9.0, 12.0])]:
        plan = backward.stamp({"x": x_gpu, "predicate_value": _scalar(value, stream), "dy": dy_gpu}, stream)
        plan.run()
        np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("x_grad"), stream), np.array(expected, np.float32), rtol=1e-6, atol=1e-6)
