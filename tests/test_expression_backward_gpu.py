"""FusedEquation.compile_backward: gradients of expression graphs, checked against closed forms and against central
differences of a float64 numpy evaluation of the forward function.  Cases and tolerances follow the reference's
bindings/python/test/core/physical/test_expression_backward_phase1.py (:115-260 elementwise subset, :1236-1500 min/max
reductions, explicit upstream gradients, name validation)."""
from __future__ import annotations

import numpy as np
import pytest
import scipy.special as sp

from helpers import FLOAT_DTYPES, copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex

pytestmark = pytest.mark.gpu

# the reference's _assert_close, test_expression_backward_phase1.py:42-56
TOLERANCE = {DataType.fp32: (1e-5, 1e-6), DataType.fp16: (5e-2, 5e-2), DataType.bf16: (5e-2, 5e-2), DataType.fp8_e4m3: (1e-1, 1e-1),
             DataType.fp8_e5m2: (2e-1, 0.5)}


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def stored(values, dtype):
    """fp32 values rounded to `dtype`, as (carrier array, float64 values the GPU sees)."""
    carrier = to_storage(np.asarray(values, np.float32), dtype)
    return carrier, from_storage(carrier, dtype).astype(np.float64)


def backward(forward, arrays, stream, wrt=None, upstream=None, dtype=DataType.fp32, dtypes=None, accumulate=False):
    """Compiles `forward` (an Expression or {name: Expression}), differentiates, binds `arrays` (name -> fp32 values, stored as
    `dtype` or dtypes[name]) and returns (plan, {output name: float64 values}, float64 inputs as the GPU sees them)."""
    fwd = ex.compile(ex.outputs(forward) if isinstance(forward, dict) else forward, device_num=0)
    bwd = fwd.compile_backward(wrt, error_input_name=upstream, accumulate_grad_outputs=accumulate)
    tensors, seen = {}, {}
    for name, values in arrays.items():
        dt = (dtypes or {}).get(name, dtype)
        carrier, seen[name] = stored(values, dt)
        tensors[name] = copy_numpy_to_gpu(carrier, stream, dt)
    plan = bwd.stamp(tensors, stream)
    plan.run()
    got = {}
    for name in bwd.output_names():
        t = plan.output(name)
        got[name] = from_storage(copy_gpu_to_numpy(t, stream), t.get_data_type()).astype(np.float64)
    return plan, got, seen, bwd


def close(got, expected, dtype):
    rtol, atol = TOLERANCE[dtype]
    np.testing.assert_allclose(got, expected, rtol=rtol, atol=atol)


# ---- the reference's elementwise subset, every float dtype ------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", FLOAT_DTYPES, ids=lambda d: d.name)
def test_supported_subset_matches_closed_forms(stream, dtype):
    x, y, z, w, v, u = (ex.input(n) for n in "xyzwvu")
    loss = ((x * y) + (x / z) - w.sqrt() + v.exp() + u.ln()).reduce_sum(axis=[0, 1], squeeze=False)
    arrays = {"x": [[1.0, 2.0, 3.0], [1.5, 2.5, 3.5]], "y": [[0.5, 1.5, 2.0], [2.5, 1.0, 0.75]], "z": [[2.0, 4.0, 5.0], [3.0, 6.0, 7.0]],
              "w": [[4.0, 9.0, 16.0], [25.0, 36.0, 49.0]], "v": [[0.1, 0.2, -0.3], [0.4, -0.2, 0.0]], "u": [[1.5, 2.0, 3.0], [4.0, 5.0, 6.0]]}
    plan, got, a, bwd = backward(loss, arrays, stream, ["x", "y", "z", "w", "v", "u"], dtype=dtype)
    assert bwd.output_names() == ["x_grad", "y_grad", "z_grad", "w_grad", "v_grad", "u_grad"]
    for name in bwd.output_names():
        assert plan.output(name).get_data_type() == dtype  # a gradient has the dtype of what it is the gradient of
        assert plan.output(name).get_dimensions() == [2, 3]
    close(got["x_grad"], a["y"] + 1 / a["z"], dtype)
    close(got["y_grad"], a["x"], dtype)
    close(got["z_grad"], -a["x"] / a["z"] ** 2, dtype)
    close(got["w_grad"], -0.5 / np.sqrt(a["w"]), dtype)
    close(got["v_grad"], np.exp(a["v"]), dtype)
    close(got["u_grad"], 1 / a["u"], dtype)
    assert plan.stage_kind_names() == ["FusedKernel"]  # six gradients, one pass


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
def test_explicit_upstream_and_broadcast_operands(stream, dtype):
    rng = np.random.default_rng(11)
    x, w, b = ex.input("x"), ex.input("w"), ex.input("b")
    arrays = {"x": rng.uniform(-2, 2, (33, 7, 20)), "w": rng.uniform(-2, 2, (7, 1)), "b": rng.uniform(-2, 2, (20,)), "__grad_output": rng.uniform(-1, 1, (33, 7, 20))}
    plan, got, a, bwd = backward(x * w + b, arrays, stream, ["x", "w", "b"], upstream="__grad_output", dtype=dtype)
    g = a["__grad_output"]
    assert [plan.output(n).get_dimensions() for n in bwd.output_names()] == [[33, 7, 20], [7, 1], [20]]
    close(got["x_grad"], g * a["w"], dtype)
    rtol, atol = TOLERANCE[dtype]
    np.testing.assert_allclose(got["w_grad"], (g * a["x"]).sum(axis=(0, 2)).reshape(7, 1), rtol=rtol, atol=atol * 30)
    np.testing.assert_allclose(got["b_grad"], g.sum(axis=(0, 1)), rtol=rtol, atol=atol * 30)


# ---- every differentiable elementwise op against central differences ---------------------------------------------------------
def _sigmoid(v):
    return 1 / (1 + np.exp(-v))


UNARY_CASES = [
    ("neg", lambda e: -e, lambda v: -v, (-2, 2)), ("abs", lambda e: e.abs(), np.abs, (0.2, 2)), ("exp", lambda e: e.exp(), np.exp, (-2, 2)),
    ("exp2", lambda e: e.exp2(), np.exp2, (-2, 2)), ("exp10", lambda e: e.exp10(), lambda v: 10.0 ** v, (-1, 1)),
    ("expm1", lambda e: e.expm1(), np.expm1, (-1, 1)), ("ln", lambda e: e.ln(), np.log, (0.3, 4)), ("log2", lambda e: e.log2(), np.log2, (0.3, 4)),
    ("log10", lambda e: e.log10(), np.log10, (0.3, 4)), ("log1p", lambda e: e.log1p(), np.log1p, (-0.5, 3)), ("sqrt", lambda e: e.sqrt(), np.sqrt, (0.3, 4)),
    ("sin", lambda e: e.sin(), np.sin, (-3, 3)), ("cos", lambda e: e.cos(), np.cos, (-3, 3)), ("tan", lambda e: e.tan(), np.tan, (-1.2, 1.2)),
    ("tanh", lambda e: e.tanh(), np.tanh, (-2, 2)), ("sinh", lambda e: e.sinh(), np.sinh, (-2, 2)), ("cosh", lambda e: e.cosh(), np.cosh, (-2, 2)),
    ("asin", lambda e: e.asin(), np.arcsin, (-0.8, 0.8)), ("acos", lambda e: e.acos(), np.arccos, (-0.8, 0.8)),
    ("atan", lambda e: e.atan(), np.arctan, (-3, 3)), ("asinh", lambda e: e.asinh(), np.arcsinh, (-3, 3)),
    ("acosh", lambda e: e.acosh(), np.arccosh, (1.3, 4)), ("atanh", lambda e: e.atanh(), np.arctanh, (-0.8, 0.8)),
    ("erf", lambda e: e.erf(), sp.erf, (-2, 2)), ("erfc", lambda e: e.erfc(), sp.erfc, (-2, 2)), ("erfcx", lambda e: e.erfcx(), sp.erfcx, (-1, 3)),
    ("erfinv", lambda e: e.erfinv(), sp.erfinv, (-0.8, 0.8)), ("erfcinv", lambda e: e.erfcinv(), sp.erfcinv, (0.2, 1.8)),
    ("normcdf", lambda e: e.normcdf(), sp.ndtr, (-2, 2)), ("lgamma", lambda e: e.lgamma(), sp.gammaln, (0.5, 4)),
    ("tgamma", lambda e: e.tgamma(), sp.gamma, (0.5, 4)), ("sigmoid", lambda e: e.sigmoid(), _sigmoid, (-3, 3)),
    ("softplus", lambda e: e.softplus(), lambda v: np.log1p(np.exp(v)), (-3, 3)), ("swish", lambda e: e.swish(), lambda v: v * _sigmoid(v), (-3, 3)),
    ("gelu", lambda e: e.gelu(), lambda v: v * sp.ndtr(v), (-3, 3)), ("relu", lambda e: e.relu(), lambda v: np.maximum(v, 0), (0.1, 2)),
    ("square via pow", lambda e: e ** 2.0, lambda v: v ** 2, (0.2, 2)), ("reciprocal", lambda e: 1.0 / e, lambda v: 1 / v, (0.4, 3)),
]


@pytest.mark.parametrize("name,build,function,domain", UNARY_CASES, ids=[c[0] for c in UNARY_CASES])
def test_unary_rules_match_central_differences(stream, name, build, function, domain):
    rng = np.random.default_rng(5)
    values = rng.uniform(domain[0], domain[1], (16, 24))
    upstream = rng.uniform(0.5, 1.5, values.shape)
    plan, got, a, _ = backward(build(ex.input("x")) * 1.0, {"x": values, "__grad_output": upstream}, stream, ["x"], upstream="__grad_output")
    h = 1e-6
    numeric = (function(a["x"] + h) - function(a["x"] - h)) / (2 * h) * a["__grad_output"]
    np.testing.assert_allclose(got["x_grad"], numeric, rtol=3e-4, atol=1e-5)
    assert plan.stage_kind_names() == ["FusedKernel"]


def test_binary_rules_pow_min_max_where(stream):
    rng = np.random.default_rng(6)
    a_values, b_values = rng.uniform(0.5, 2.0, (40, 9)), rng.uniform(0.5, 2.0, (40, 9))
    b_values[::5] = a_values[::5]  # ties: min/max split the gradient evenly
    x, y = ex.input("x"), ex.input("y")
    forward = {"p": x ** y, "lo": x.min(y), "hi": x.max(y), "pick": ex.where(x > 1.2, x * y, y - x)}
    ups = {"p": "__gp", "lo": "__glo", "hi": "__ghi", "pick": "__gpick"}
    arrays = {"x": a_values, "y": b_values}
    arrays.update({u: rng.uniform(0.5, 1.5, (40, 9)) for u in ups.values()})
    _, got, a, _ = backward(forward, arrays, stream, ["x", "y"], upstream=ups)
    xv, yv = a["x"], a["y"]
    left = np.where(xv < yv, 1.0, np.where(xv > yv, 0.0, 0.5))
    cond = xv > 1.2
    expected_x = (a["__gp"] * yv * xv ** (yv - 1) + a["__glo"] * left + a["__ghi"] * (1 - left) + a["__gpick"] * np.where(cond, yv, -1.0))
    expected_y = (a["__gp"] * xv ** yv * np.log(xv) + a["__glo"] * (1 - left) + a["__ghi"] * left + a["__gpick"] * np.where(cond, xv, 1.0))
    np.testing.assert_allclose(got["x_grad"], expected_x, rtol=2e-5, atol=1e-6)
    np.testing.assert_allclose(got["y_grad"], expected_y, rtol=2e-5, atol=1e-6)


# ---- reductions -------------------------------------------------------------------------------------------------------------------
REDUCTION_SHAPES = [((6, 5, 4), [1], False), ((6, 5, 4), [1], True), ((6, 5, 4), [0, 2], [0, 2]), ((6, 5, 4), None, False), ((37, 130), [1], [1]), ((37, 130), [0], True)]


@pytest.mark.parametrize("shape,axis,squeeze", REDUCTION_SHAPES, ids=str)
@pytest.mark.parametrize("op", ["reduce_sum", "reduce_mean", "reduce_prod", "reduce_norm1", "reduce_norm2"])
def test_value_reductions(stream, op, shape, axis, squeeze):
    rng = np.random.default_rng(8)
    values = rng.uniform(0.6, 1.4, shape) * rng.choice([-1.0, 1.0], shape)
    axes = tuple(range(len(shape))) if axis is None else tuple(axis)
    out = {"reduce_sum": np.sum, "reduce_mean": np.mean, "reduce_prod": np.prod, "reduce_norm1": lambda v, **k: np.abs(v).sum(**k),
           "reduce_norm2": lambda v, **k: np.sqrt((v * v).sum(**k))}[op](values, axis=axes, keepdims=True)
    keep = squeeze is False
    out_shape = out.shape if keep else tuple(d for i, d in enumerate(out.shape) if not ((squeeze is True and d == 1) or (squeeze is not True and i in squeeze)))
    upstream = rng.uniform(0.5, 1.5, out_shape if out_shape else (1,))
    forward = getattr(ex.input("x"), op)(axis=axis, squeeze=squeeze)
    _, got, a, _ = backward(forward, {"x": values, "__grad_output": upstream}, stream, ["x"], upstream="__grad_output")
    v = a["x"]
    g = a["__grad_output"].reshape(out.shape)
    count = np.prod([shape[i] for i in axes])
    expected = {"reduce_sum": lambda: g * np.ones_like(v), "reduce_mean": lambda: g / count * np.ones_like(v),
                "reduce_prod": lambda: g * np.prod(v, axis=axes, keepdims=True) / v, "reduce_norm1": lambda: g * np.sign(v),
                "reduce_norm2": lambda: g * v / np.sqrt((v * v).sum(axis=axes, keepdims=True))}[op]()
    np.testing.assert_allclose(got["x_grad"], expected, rtol=5e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("op", ["reduce_min", "reduce_max"])
@pytest.mark.parametrize("shape,axis,squeeze", REDUCTION_SHAPES + [((2, 3), [0, 1], False), ((3000, 33), [0], [0])], ids=str)
def test_min_max_reductions_route_to_the_first_winner(stream, op, shape, axis, squeeze, dtype):
    rng = np.random.default_rng(9)
    values = np.round(rng.uniform(-4, 4, shape) * 2) / 2  # half-integers: exact in every dtype, many ties
    axes = tuple(range(len(shape))) if axis is None else tuple(axis)
    kept = [i for i in range(len(shape)) if i not in axes]
    moved = np.transpose(values, kept + list(axes)).reshape(int(np.prod([shape[i] for i in kept])) if kept else 1, -1)
    winner = (np.argmin if op == "reduce_min" else np.argmax)(moved, axis=1)  # numpy picks the first among equals too
    upstream = rng.uniform(0.5, 1.5, moved.shape[0])
    keepdims_shape = tuple(1 if i in axes else d for i, d in enumerate(shape))
    if squeeze is False:
        up_shape = keepdims_shape
    elif squeeze is True:
        up_shape = tuple(d for d in keepdims_shape if d != 1) or (1,)
    else:
        up_shape = tuple(d for i, d in enumerate(keepdims_shape) if i not in squeeze) or (1,)
    forward = getattr(ex.input("x"), op)(axis=axis, squeeze=squeeze)
    plan, got, a, _ = backward(forward, {"x": values, "__grad_output": upstream.reshape(up_shape)}, stream, ["x"], upstream="__grad_output", dtype=dtype)
    routed = np.zeros_like(moved)
    routed[np.arange(moved.shape[0]), winner] = a["__grad_output"].reshape(-1)
    inverse = np.argsort(kept + list(axes))
    expected = np.transpose(routed.reshape([shape[i] for i in kept] + [shape[i] for i in axes]), inverse)
    np.testing.assert_array_equal(got["x_grad"], expected)  # values are copied, never computed: exact
    assert plan.output("x_grad").get_data_type() == dtype
    assert plan.stage_kind_names()[-2:] == ["ArgMinMax", "ReduceMinMaxBackward"]


def test_reduce_min_tie_uses_first_logical_index(stream):
    """test_expression_backward_phase1.py:1277-1312 there."""
    values = np.array([[3.0, 1.0, 1.0, 2.0], [0.5, 0.5, 0.5, 0.5]])
    _, got, _, _ = backward(ex.input("x").reduce_min(axis=1, squeeze=[1]), {"x": values}, stream, ["x"])
    np.testing.assert_array_equal(got["x_grad"], [[0, 1, 0, 0], [1, 0, 0, 0]])


def test_min_max_of_a_computed_value_feed_further_arithmetic(stream):
    rng = np.random.default_rng(10)
    values = rng.uniform(-2, 2, (50, 70))
    x = ex.input("x")
    spread = (x.exp().reduce_max(axis=1) - (x * x).reduce_min(axis=1)).reduce_sum(axis=[0, 1])  # sum over rows of max(e^x) - min(x^2)
    _, got, a, _ = backward(spread, {"x": values}, stream, ["x"])
    v = a["x"]
    expected = np.zeros_like(v)
    rows = np.arange(v.shape[0])
    hi, lo = np.argmax(np.exp(v), axis=1), np.argmin(v * v, axis=1)
    expected[rows, hi] += np.exp(v[rows, hi])
    expected[rows, lo] -= 2 * v[rows, lo]
    np.testing.assert_allclose(got["x_grad"], expected, rtol=2e-6, atol=1e-7)


# ---- softmax, shape ops, casts ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("log", [False, True], ids=["softmax", "log_softmax"])
@pytest.mark.parametrize("shape", [(64, 10), (33, 1000), (8, 16, 5)], ids=str)
def test_softmax_backward_is_one_row_kernel(stream, shape, log, dtype):
    rng = np.random.default_rng(12)
    values, upstream = rng.uniform(-3, 3, shape), rng.uniform(-1, 1, shape)
    x = ex.input("x")
    plan, got, a, _ = backward(x.log_softmax() if log else x.softmax(), {"x": values, "__grad_output": upstream}, stream, ["x"], upstream="__grad_output", dtype=dtype)
    v, g = a["x"], a["__grad_output"]
    e = np.exp(v - v.max(axis=1, keepdims=True))
    p = e / e.sum(axis=1, keepdims=True)
    expected = g - p * g.sum(axis=1, keepdims=True) if log else p * (g - (g * p).sum(axis=1, keepdims=True))
    rtol, atol = TOLERANCE[dtype]
    np.testing.assert_allclose(got["x_grad"], expected, rtol=rtol * 4, atol=atol)
    if len(shape) == 2:
        assert plan.stage_kind_names() == ["FusedRowKernel"]  # the forward probabilities are recomputed in registers


def test_shape_ops_and_transposes(stream):
    rng = np.random.default_rng(13)
    values, weights = rng.uniform(-2, 2, (6, 20)), rng.uniform(-2, 2, (20, 6))
    x, w = ex.input("x"), ex.input("w")
    forward = {"a": x.reshape([3, 40]).exp(), "b": (x.transpose() * w).tanh(), "c": x.unsqueeze([1]).squeeze([1]) * 3.0}
    ups = {"a": "__ga", "b": "__gb", "c": "__gc"}
    arrays = {"x": values, "w": weights, "__ga": rng.uniform(-1, 1, (3, 40)), "__gb": rng.uniform(-1, 1, (20, 6)), "__gc": rng.uniform(-1, 1, (6, 20))}
    _, got, a, _ = backward(forward, arrays, stream, ["x", "w"], upstream=ups)
    v, wv = a["x"], a["w"]
    t = np.tanh(v.T * wv)
    expected_x = (a["__ga"] * np.exp(v.reshape(3, 40))).reshape(6, 20) + (a["__gb"] * (1 - t * t) * wv).T + 3 * a["__gc"]
    np.testing.assert_allclose(got["x_grad"], expected_x, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got["w_grad"], a["__gb"] * (1 - t * t) * v.T, rtol=1e-5, atol=1e-6)


def test_casts_pass_gradients_straight_through_in_the_operand_dtype(stream):
    rng = np.random.default_rng(14)
    h, f = ex.input("h"), ex.input("f")
    arrays = {"h": rng.uniform(-2, 2, (30, 12)), "f": rng.uniform(-2, 2, (30, 12))}
    plan, got, a, _ = backward((h.cast(DataType.fp32) * f).reduce_sum(axis=[0, 1]), arrays, stream, ["h", "f"], dtypes={"h": DataType.fp16})
    assert plan.output("h_grad").get_data_type() == DataType.fp16 and plan.output("f_grad").get_data_type() == DataType.fp32
    close(got["h_grad"], a["f"], DataType.fp16)
    close(got["f_grad"], a["h"], DataType.fp32)


# ---- several outputs, shared and absent gradients, accumulation ---------------------------------------------------------------
def test_multi_output_upstream_map_may_be_partial(stream):
    rng = np.random.default_rng(15)
    x, w = ex.input("x"), ex.input("w")
    forward = {"main": x * w, "aux": x.exp(), "unused": w.ln()}
    arrays = {"x": rng.uniform(0.5, 2, (9, 8)), "w": rng.uniform(0.5, 2, (9, 8)), "__grad_main": rng.uniform(-1, 1, (9, 8)), "__grad_aux": rng.uniform(-1, 1, (9, 8))}
    _, got, a, bwd = backward(forward, arrays, stream, ["x", "w"], upstream={"main": "__grad_main", "aux": "__grad_aux"})
    assert bwd.output_names() == ["x_grad", "w_grad"]
    np.testing.assert_allclose(got["x_grad"], a["__grad_main"] * a["w"] + a["__grad_aux"] * np.exp(a["x"]), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got["w_grad"], a["__grad_main"] * a["x"], rtol=1e-5, atol=1e-6)


def test_equal_and_absent_gradients_get_tensors_of_their_own(stream):
    rng = np.random.default_rng(16)
    x, c, d = ex.input("x"), ex.input("c"), ex.input("d")
    arrays = {"x": rng.uniform(-1, 1, (5, 6)), "c": rng.uniform(-1, 1, (5, 6)), "d": rng.uniform(-1, 1, (5, 6)), "__grad_output": rng.uniform(-1, 1, (5, 6))}
    forward = {"y": x + c, "z": d * 2.0}
    plan, got, a, _ = backward(forward, arrays, stream, ["x", "c", "d"], upstream={"y": "__grad_output"})
    np.testing.assert_array_equal(got["x_grad"], a["__grad_output"])
    np.testing.assert_array_equal(got["c_grad"], a["__grad_output"])
    np.testing.assert_array_equal(got["d_grad"], np.zeros((5, 6)))  # no upstream gradient reaches d
    assert plan.output("x_grad").mem_ptr() != plan.output("c_grad").mem_ptr()


def test_accumulate_adds_to_the_running_gradients(stream):
    rng = np.random.default_rng(17)
    x, w = ex.input("x"), ex.input("w")
    arrays = {"x": rng.uniform(-1, 1, (12, 4)), "w": rng.uniform(-1, 1, (4,)), "x_grad": rng.uniform(-1, 1, (12, 4)), "w_grad": rng.uniform(-1, 1, (4,))}
    _, got, a, _ = backward((x * w).reduce_sum(axis=[0, 1]), arrays, stream, ["x", "w"], accumulate=True)
    np.testing.assert_allclose(got["x_grad"], a["x_grad"] + a["w"] * np.ones((12, 1)), rtol=1e-6)
    np.testing.assert_allclose(got["w_grad"], a["w_grad"] + a["x"].sum(axis=0), rtol=1e-5, atol=1e-6)


def test_backward_equations_specialise_per_shape_and_reuse_kernels(stream):
    x = ex.input("x")
    bwd = ex.compile((x * x).reduce_sum(axis=1), device_num=0).compile_backward(["x"])
    for rows in (8, 8, 20):
        values = np.arange(rows * 6, dtype=np.float32).reshape(rows, 6)
        plan = bwd.stamp({"x": copy_numpy_to_gpu(values, stream, DataType.fp32)}, stream)
        plan.run()
        np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("x_grad"), stream), 2 * values)
    again = ph.compiled_kernel_count()
    bwd.stamp({"x": copy_numpy_to_gpu(np.ones((8, 6), np.float32), stream, DataType.fp32)}, stream)
    assert ph.compiled_kernel_count() == again  # a shape seen before compiles nothing
    assert bwd.get_output_shape({"x": copy_numpy_to_gpu(np.ones((3, 6), np.float32), stream, DataType.fp32)}, "x_grad") == ([3, 6], DataType.fp32)


# ---- ragged batches -----------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("mean", [False, True], ids=["sum", "mean"])
def test_segmented_reductions_and_broadcasts(stream, mean):
    rng = np.random.default_rng(18)
    capacity, width = 700, 16
    offsets = np.array([0, 120, 120, 400, 401, 650], np.uint32)
    segments = len(offsets) - 1
    values, per_segment = rng.uniform(-1, 1, (capacity, width)), rng.uniform(-1, 1, (segments, width))
    v, s, off = ex.input("v"), ex.input("s"), ex.input("off")
    reduce = v.segment_mean(off) if mean else v.segment_sum(off)
    forward = {"reduced": reduce.exp(), "spread": s.segmented_broadcast(off, segments, capacity, width, normalize_by_segment_length=mean) * v}
    ups = {"reduced": "__gr", "spread": "__gs"}
    fwd = ex.compile(ex.outputs(forward), device_num=0)
    bwd = fwd.compile_backward(["v", "s"], error_input_name=ups)
    gr, gs = rng.uniform(-1, 1, (segments, width)).astype(np.float32), rng.uniform(-1, 1, (capacity, width)).astype(np.float32)
    tensors = {"v": copy_numpy_to_gpu(values.astype(np.float32), stream, DataType.fp32), "s": copy_numpy_to_gpu(per_segment.astype(np.float32), stream, DataType.fp32),
               "off": copy_numpy_to_gpu(offsets, stream, DataType.uint32), "__gr": copy_numpy_to_gpu(gr, stream, DataType.fp32),
               "__gs": copy_numpy_to_gpu(gs, stream, DataType.fp32)}
    plan = bwd.stamp(tensors, stream)
    plan.run()
    got_v, got_s = copy_gpu_to_numpy(plan.output("v_grad"), stream).astype(np.float64), copy_gpu_to_numpy(plan.output("s_grad"), stream).astype(np.float64)
    values, per_segment = values.astype(np.float32).astype(np.float64), per_segment.astype(np.float32).astype(np.float64)
    expected_v, expected_s = np.zeros_like(values), np.zeros_like(per_segment)
    for b in range(segments):
        lo, hi = int(offsets[b]), int(offsets[b + 1])
        n = hi - lo
        if n == 0:
            continue
        rows = values[lo:hi]
        reduced = rows.mean(axis=0) if mean else rows.sum(axis=0)
        scale = 1.0 / n if mean else 1.0
        expected_v[lo:hi] = gr[b] * np.exp(reduced) * scale + gs[lo:hi] * per_segment[b] * scale
        expected_s[b] = (gs[lo:hi] * rows).sum(axis=0) * scale
    active = int(offsets[-1])
    np.testing.assert_allclose(got_v[:active], expected_v[:active], rtol=2e-5, atol=2e-6)  # rows past the partition are padding
    np.testing.assert_allclose(got_s, expected_s, rtol=2e-5, atol=2e-6)
    with pytest.raises(RuntimeError, match="offsets are metadata and are not differentiable"):
        fwd.compile_backward(["off"], error_input_name=ups).stamp(tensors, stream)


# ---- validation (messages of AutoDiff.cpp:2486-2581 there) -----------------------------------------------------------------------
def test_name_validation(stream):
    x, y = ex.input("x"), ex.input("y")
    fwd = ex.compile(x * y, device_num=0)
    with pytest.raises(RuntimeError, match="collides with an existing forward input"):
        fwd.compile_backward(["x"], error_input_name="y")
    with pytest.raises(RuntimeError, match="Requested gradient for unknown input: nope"):
        fwd.compile_backward(["nope"])
    with pytest.raises(RuntimeError, match="Duplicate wrt input name"):
        fwd.compile_backward(["x", "x"])
    with pytest.raises(RuntimeError, match="explicit upstream input name cannot be empty"):
        fwd.compile_backward(["x"], error_input_name="")
    with pytest.raises(RuntimeError, match="Cannot compute backward expression with no error inputs"):
        fwd.compile_backward(["x"], error_input_name={})
    with pytest.raises(RuntimeError, match="unknown forward output"):
        fwd.compile_backward(["x"], error_input_name={"elsewhere": "__g"})
    scaled = ex.compile(x * ex.runtime_scalar("alpha"), device_num=0)
    with pytest.raises(RuntimeError, match="only supports gradients with respect to tensor inputs"):
        scaled.compile_backward(["alpha"])
    two = ex.compile(ex.outputs({"a": x + y, "b": x - y}), device_num=0)
    with pytest.raises(RuntimeError, match="requires an explicit upstream seed map"):
        two.compile_backward(["x"])
    with pytest.raises(RuntimeError, match="only supports exactly one forward output"):
        two.compile_backward(["x"], error_input_name="__g")
    assert fwd.compile_backward().output_names() == ["x_grad", "y_grad"]  # no names: every tensor input
    ones = copy_numpy_to_gpu(np.ones((4, 4), np.float32), stream, DataType.fp32)
    with pytest.raises(RuntimeError, match="Missing required input tensor: y"):
        fwd.compile_backward(["x"]).stamp({"x": ones}, stream)
    with pytest.raises(RuntimeError, match="Unexpected input tensor for this equation: z"):
        fwd.compile_backward(["x"]).stamp({"x": ones, "y": ones, "z": ones}, stream)
    with pytest.raises(RuntimeError, match="does not support backward for op floor"):
        ex.compile(x.floor() * y, device_num=0).compile_backward(["x"]).stamp({"x": ones, "y": ones}, stream)
    # a runtime scalar flows through the backward equation like any other operand
    plan = scaled.compile_backward(["x"]).stamp({"x": ones}, stream)
    plan.run({"alpha": 2.5})
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("x_grad"), stream), np.full((4, 4), 2.5, np.float32))
