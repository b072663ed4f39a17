"""Host side of the path, no GPU needed: Expression DAG building and canonical text, dtype resolution, shape inference and
the CPU TypeConverter, against the reference's rules (Utilities/Expression/Expression.cpp:3261-3296 activation decompositions,
ExpressionDTypeResolution.cpp:277-307 promotion, StampedEquation.h:460-462 + SqueezeAxes.cpp output dims,
Utilities/TensorOperations/DataTypeConversions/TypeConverter.cpp:899-942 cpuConvertTypeImpl)."""
from __future__ import annotations

import numpy as np
import pytest

import oracle
from thor_amd import physical as ph
from thor_amd.dtypes import DataType as D, numpy_carrier
from thor_amd.physical import Expression as ex


def cpu(shape, dtype):
    return ph.PhysicalTensor(ph.Placement(ph.DeviceType.cpu, 0), ph.PhysicalTensor.Descriptor(dtype, list(shape)))


def out(expr, **inputs):
    return ex.compile(expr, 0).get_output_shape(inputs)


def test_sigmoid_lowers_to_the_overflow_safe_decomposition():
    """sigmoid(d) = exp(-max(-d, 0)) / (1 + exp(-|d|)) (Expression.cpp:3261-3296)."""
    s = ex.input("d").sigmoid()
    assert s.canonical() == "div(exp(neg(max(neg(input#0),scalar(0)))),add(exp(neg(abs(input#0))),scalar(1)))"
    config1 = (ex.input("a") * ex.input("b") + ex.input("c")) * ex.input("d").sigmoid()
    text = config1.canonical()
    # commutative operands print in canonical order, so a*b+c appears as add(c, mul(a, b))
    assert text == ("mul(add(input#2,mul(input#0,input#1)),"
                    "div(exp(neg(max(neg(input#3),scalar(0)))),add(exp(neg(abs(input#3))),scalar(1))))")


def test_commutative_operands_are_ordered_and_equal_graphs_print_equally():
    a, b = ex.input("a"), ex.input("b")
    assert (a + b).canonical() == (b + a).canonical()
    assert (a * b).canonical() == (b * a).canonical()
    assert (a - b.exp()).canonical() != (b.exp() - a).canonical()  # subtraction keeps its operand order
    e1 = (a * 2.0 + b).tanh()
    e2 = (ex.input("a") * 2.0 + ex.input("b")).tanh()
    assert e1.canonical() == e2.canonical()


PROMOTION = [(D.fp16, D.fp16, D.fp16), (D.bf16, D.bf16, D.bf16), (D.fp16, D.bf16, D.fp32), (D.fp32, D.fp16, D.fp32), (D.fp32, D.bf16, D.fp32),
             (D.fp8_e4m3, D.fp8_e4m3, D.fp8_e4m3), (D.fp8_e4m3, D.fp8_e5m2, D.fp16), (D.fp8_e5m2, D.bf16, D.bf16), (D.fp8_e4m3, D.fp16, D.fp16),
             (D.int32, D.int32, D.int32), (D.uint32, D.uint32, D.uint32)]


@pytest.mark.parametrize("da,db,want", PROMOTION, ids=lambda v: v.name)
def test_binary_promotion_follows_the_reference_table(da, db, want):
    """ExpressionDTypeResolution.cpp:277-307: equal types stay; fp16 with bf16 -> fp32; anything with fp32 -> fp32;
    bf16 beats fp16-less partners; two different fp8 types -> fp16."""
    shape, dtype = out(ex.input("a") + ex.input("b"), a=cpu([3], da), b=cpu([3], db))
    assert shape == [3] and dtype == want
    shape, dtype = out(ex.input("b") * ex.input("a"), a=cpu([3], da), b=cpu([3], db))
    assert dtype == want


def test_mixing_integer_and_floating_tensors_is_rejected_like_the_reference():
    with pytest.raises(RuntimeError, match="Unsupported dtype in promoteTensorValueDTypes"):
        out(ex.input("a") + ex.input("b"), a=cpu([3], D.uint8), b=cpu([3], D.fp16))
    with pytest.raises(RuntimeError, match="Unsupported dtype in promoteTensorValueDTypes"):
        out(ex.input("a") * ex.input("b"), a=cpu([3], D.int32), b=cpu([3], D.fp32))


@pytest.mark.parametrize("dtype", [D.fp16, D.bf16, D.fp8_e4m3, D.fp8_e5m2, D.fp32, D.int32], ids=lambda d: d.name)
def test_reductions_default_to_fp32_and_arg_reductions_to_uint32(dtype):
    a = ex.input("a")
    assert out(a.reduce_sum(axis=0), a=cpu([3, 4], dtype)) == ([1, 4], D.fp32)
    assert out(a.reduce_mean(axis=1, squeeze=True), a=cpu([3, 4], dtype)) == ([3], D.fp32)
    assert out(a.reduce_max(axis=0, output_dtype=D.bf16), a=cpu([3, 4], dtype))[1] == D.bf16
    assert out(a.argmin(axis=1, squeeze=True), a=cpu([3, 4], dtype)) == ([3], D.uint32)
    assert out(a.argmax(axis=1), a=cpu([3, 4], dtype)) == ([3, 1], D.uint32)


def test_scalars_do_not_promote_and_casts_do():
    a = ex.input("a")
    assert out(a * 2.0, a=cpu([3], D.int32))[1] == D.int32
    assert out(a * 2.0, a=cpu([3], D.fp16))[1] == D.fp16
    assert out(a.cast(D.fp16) * 2.0, a=cpu([3], D.int32))[1] == D.fp16
    assert out(a.exp(), a=cpu([3], D.fp8_e4m3))[1] == D.fp8_e4m3
    assert out(a < ex.input("b"), a=cpu([3], D.fp32), b=cpu([3], D.fp32)) == ([3], D.boolean)
    assert out(a.with_output_dtype(D.bf16) + 1.0, a=cpu([3], D.fp32))[1] in (D.bf16, D.fp32)


def test_shapes_numpy_broadcasting_squeeze_and_views():
    a, b = ex.input("a"), ex.input("b")
    assert out(a + b, a=cpu([4, 1, 5], D.fp32), b=cpu([3, 1], D.fp32))[0] == [4, 3, 5]
    assert out(a + b, a=cpu([4, 5], D.fp32), b=cpu([5], D.fp32))[0] == [4, 5]
    assert out((a * b).reduce_sum(axis=[0, 2], squeeze=[0]), a=cpu([2, 3, 4], D.fp16), b=cpu([4], D.fp16)) == ([3, 1], D.fp32)
    assert out(a.reduce_sum(axis=None, squeeze=True), a=cpu([2, 3, 4], D.fp32))[0] == [1]
    assert out(a.reduce_sum(axis=None), a=cpu([2, 3, 4], D.fp32))[0] == [1, 1, 1]
    assert out(a.reshape([2, 6]), a=cpu([3, 4], D.fp32))[0] == [2, 6]
    assert out(a.unsqueeze([0, 3]), a=cpu([3, 4], D.fp32))[0] == [1, 3, 4, 1]
    assert out(a.unsqueeze([1]).squeeze([1]), a=cpu([3, 4], D.fp32))[0] == [3, 4]
    with pytest.raises(RuntimeError, match="broadcast"):
        out(a + b, a=cpu([3, 4], D.fp32), b=cpu([5], D.fp32))
    with pytest.raises(RuntimeError, match="axis"):
        out(a.reduce_sum(axis=3), a=cpu([3, 4], D.fp32))
    with pytest.raises(RuntimeError, match="squeeze"):
        out(a.squeeze([0]), a=cpu([3, 4], D.fp32))
    with pytest.raises(RuntimeError, match="Missing required input"):
        out(a + b, a=cpu([3], D.fp32))


def test_named_outputs_and_their_dtypes():
    a = ex.input("a")
    eq = ex.compile(ex.outputs({"soft": a.exp() / a.exp().reduce_sum(axis=1), "best": a.argmax(axis=1, squeeze=True), "half": a.cast(D.fp16)}), 0)
    assert sorted(eq.output_names()) == ["best", "half", "soft"]
    ins = {"a": cpu([6, 7], D.bf16)}
    assert eq.get_output_shape(ins, "soft") == ([6, 7], D.fp32)  # bf16 / fp32 row sum promotes to fp32
    assert eq.get_output_shape(ins, "best") == ([6], D.uint32)
    assert eq.get_output_shape(ins, "half") == ([6, 7], D.fp16)


# ---- CPU TypeConverter (the reference's only in-tree CPU path) ---------------------------------------------------------------------
FLOATS = [D.fp16, D.bf16, D.fp8_e4m3, D.fp8_e5m2, D.fp32, D.fp64]
INTS = [D.int8, D.int16, D.int32, D.int64, D.uint8, D.uint16, D.uint32, D.uint64, D.boolean]


def sample(dtype, n, rng):
    if dtype in (D.fp32, D.fp64):
        x = rng.standard_normal(n) * 50
        x[::97] *= 1e5
        x[1::97] *= 1e-7
        x[5::1001] = 0
        return x.astype(numpy_carrier(dtype))
    if dtype in FLOATS:
        x = (rng.standard_normal(n) * 20).astype(np.float32)
        return oracle.convert(x, oracle.FP32, int(dtype))
    if dtype == D.boolean:
        return rng.integers(0, 2, n).astype(np.uint8)
    info = np.iinfo(numpy_carrier(dtype))
    return rng.integers(max(info.min, -100), min(info.max, 100), n, dtype=np.int64).astype(numpy_carrier(dtype))


@pytest.mark.parametrize("src", FLOATS + INTS, ids=lambda d: d.name)
def test_cpu_type_converter_matches_the_oracle_for_every_destination(src):
    rng = np.random.default_rng(int(src))
    x = sample(src, 70_001, rng)
    with pytest.raises(ValueError, match="two different dtypes"):
        ph.convert_type_cpu(x, src, src)
    for dst in FLOATS + INTS:
        if dst == src:
            continue
        if src in (D.fp32, D.fp64) and dst in INTS:
            values = np.abs(x) % 100 if dst in (D.uint8, D.uint16, D.uint32, D.uint64, D.boolean) else np.clip(x, -100, 100)
            values = values.astype(x.dtype)
        else:
            values = x
        if src in FLOATS and src not in (D.fp32, D.fp64) and dst in (D.uint8, D.uint16, D.uint32, D.uint64):
            values = oracle.convert(np.abs(oracle.convert(values, int(src), oracle.FP32)), oracle.FP32, int(src))
        got = ph.convert_type_cpu(values, src, dst)
        want = oracle.convert(values, int(src), int(dst))
        assert got.dtype == want.dtype
        np.testing.assert_array_equal(got.view(np.uint8), want.view(np.uint8), err_msg=f"{src.name}->{dst.name}")


def test_cpu_type_converter_large_buffer_uses_the_thread_partition_and_stays_exact():
    """n / 500000 worker ranges (TypeConverter.cpp:899-942): results must not depend on the partition."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal(3_300_017).astype(np.float32)
    x[::100] *= np.float32(1e5)
    x[1::100] *= np.float32(1e-40)
    for dst in (D.fp16, D.bf16):
        got = ph.convert_type_cpu(x, D.fp32, dst)
        want = oracle.convert(x, oracle.FP32, int(dst))
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
        back = ph.convert_type_cpu(got, dst, D.fp32)
        np.testing.assert_array_equal(back.view(np.uint32), oracle.convert(want, int(dst), oracle.FP32).view(np.uint32))


def test_conditional_outputs_validate_their_branches_like_the_reference():
    """Outputs::conditional / ifElifElse argument checks (Expression.cpp:5342-5390 there; test_expression_outputs.py:597-622)."""
    x, selector = ex.input("x"), ex.input("selector")
    then_outputs, else_outputs = ex.outputs({"y": x + 10.0}), ex.outputs({"y": x + 40.0})
    with pytest.raises(RuntimeError, match="requires at least one elif branch"):
        ex.if_elif_else(selector > 2.0, then_outputs, [], else_outputs)
    with pytest.raises(RuntimeError, match="same output names in the same order"):
        ex.if_else(selector > 0.0, then_outputs, ex.outputs({"z": x}))
    with pytest.raises(RuntimeError, match="same output names in the same order"):
        ex.if_else(selector > 0.0, ex.outputs({"a": x, "b": x * 2.0}), ex.outputs({"b": x, "a": x}))
    chained = ex.if_elif_else(selector > 2.0, then_outputs, [(selector > 1.0, ex.outputs({"y": x + 20.0})), (selector > 0.0, ex.outputs({"y": x + 30.0}))],
                              else_outputs)
    shape, dtype = chained.compile(0).get_output_shape({"x": cpu([4, 5], D.fp32), "selector": cpu([1], D.fp32)}, "y")
    assert shape == [4, 5] and dtype == D.fp32
