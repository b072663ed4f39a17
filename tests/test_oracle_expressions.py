"""Pins the host restatements of the BASELINE expression workloads (oracle/thor_oracle_expr.c) against float64 closed forms
and, for the fp16 paths, against numpy's IEEE float16 arithmetic bit for bit."""
from __future__ import annotations

import numpy as np

import oracle
from helpers import ulp_distance_f32


def test_config1_expression_within_a_few_ulp_of_the_closed_form():
    rng = np.random.default_rng(1234)
    a, b, c, d = (rng.uniform(-1, 1, 100_003).astype(np.float32) for _ in range(4))
    d[:7] = [-200.0, -88.0, -20.0, 0.0, 20.0, 88.0, 200.0]  # the decomposition must not overflow at either end
    got, threads = oracle.expr_config1(a, b, c, d)
    assert threads >= 1
    a64, b64, c64, d64 = (v.astype(np.float64) for v in (a, b, c, d))
    sig = 1.0 / (1.0 + np.exp(-d64))
    want = (a64 * b64 + c64) * sig
    # a*b and +c round separately and the sigmoid is two expf, an add and a divide: 4 ulp of the result plus the rounding of the
    # (possibly cancelling) sum
    bound = 4 * np.spacing(np.abs(want).astype(np.float32)).astype(np.float64) + np.spacing(np.maximum(np.abs(a64 * b64), np.abs(c64)).astype(np.float32)) * sig
    normal = np.abs(want) >= 1e-30  # results in the subnormal range only have to be tiny and finite
    assert np.all(np.abs(got.astype(np.float64) - want)[normal] <= bound[normal])
    assert np.all(np.abs(got[~normal]) < 1e-29)
    assert np.isfinite(got[:7]).all()


def test_softmax_rows_bf16_and_normalize_rows():
    rng = np.random.default_rng(1237)
    x = (rng.standard_normal((37, 1000)) * 3).astype(np.float32)
    bits = oracle.convert(x, oracle.FP32, oracle.BF16)
    got, _ = oracle.softmax_rows_bf16(bits)
    xb = oracle.convert(bits, oracle.BF16, oracle.FP32).astype(np.float64)
    p = np.exp(xb - xb.max(axis=1, keepdims=True))
    np.testing.assert_allclose(got, p / p.sum(axis=1, keepdims=True), rtol=3e-6, atol=1e-12)
    np.testing.assert_allclose(got.astype(np.float64).sum(axis=1), 1.0, rtol=1e-5)
    y = (rng.standard_normal((64, 1024)) * 4 + 1).astype(np.float32)
    got, _ = oracle.normalize_rows_f32(y, 1e-5)
    y64 = y.astype(np.float64)
    mu = y64.mean(axis=1, keepdims=True)
    want = (y64 - mu) / np.sqrt(((y64 - mu) ** 2).mean(axis=1, keepdims=True) + 1e-5)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6)


def test_softmax_and_normalize_at_the_row_lengths_of_the_baseline_config():
    """Rows of 4 096 bf16 (softmax) and 1 024 fp32 (normalise), the lengths the full-size GPU comparison runs on: the fp32
    row sums of the restatement (pairwise) stay within 3e-6 of the float64 closed form there, and every softmax row sums
    to one."""
    rng = np.random.default_rng(1239)
    x = (rng.standard_normal((48, 4096)) * 3).astype(np.float32)
    x[0] = 0.0  # a flat row: every probability is 1/4096 exactly
    x[1, :] = -30.0
    x[1, 77] = 30.0  # one dominant element: the others underflow towards 0 without disturbing the sum
    bits = oracle.convert(x, oracle.FP32, oracle.BF16)
    got, _ = oracle.softmax_rows_bf16(bits)
    xb = oracle.convert(bits, oracle.BF16, oracle.FP32).astype(np.float64)
    p = np.exp(xb - xb.max(axis=1, keepdims=True))
    want = p / p.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(got, want, rtol=3e-6, atol=1e-30)
    np.testing.assert_array_equal(got[0], np.full(4096, 1.0 / 4096, np.float32))
    assert got[1, 77] == 1.0
    np.testing.assert_allclose(got.astype(np.float64).sum(axis=1), 1.0, rtol=2e-6)
    y = (rng.standard_normal((96, 1024)) * 4 + 1).astype(np.float32)
    got, _ = oracle.normalize_rows_f32(y, 1e-5)
    y64 = y.astype(np.float64)
    mu = y64.mean(axis=1, keepdims=True)
    want = (y64 - mu) / np.sqrt(((y64 - mu) ** 2).mean(axis=1, keepdims=True) + 1e-5)
    # x - mean cancels near the mean: the absolute term is a few fp32 roundings of |x| ~ 16 divided by sigma ~ 4
    np.testing.assert_allclose(got, want, rtol=3e-6, atol=3e-6)


def test_fp16_relu_scale_bias_is_bit_exact_with_ieee_half_arithmetic_and_stats_accumulate_in_fp32():
    rng = np.random.default_rng(1238)
    x = rng.standard_normal((3, 8, 5, 7)).astype(np.float16)
    scale = rng.uniform(0.5, 1.5, 8).astype(np.float16)
    bias = rng.uniform(-0.1, 0.1, 8).astype(np.float16)
    got, _ = oracle.relu_scale_bias_f16(x, scale, bias)
    s, b = scale.reshape(1, 8, 1, 1), bias.reshape(1, 8, 1, 1)
    want = np.maximum((x * s).astype(np.float16) + b, np.float16(0)).astype(np.float16)  # numpy rounds after each half operation
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    total, squares, _ = oracle.channel_stats_f16(x)
    np.testing.assert_allclose(total, x.astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(squares, (x * x).astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-5)


def test_rows_sum_max_argmax_with_ties_and_nans():
    x = np.array([[5.0, 5.0, 3.0, 5.0], [-1.0, np.nan, np.nan, 8.0], [1.0, 2.0, 3.0, 3.0]], dtype=np.float32)
    s, m, a, _ = oracle.rows_f32(x)
    assert a.tolist() == [0, 1, 2]
    assert m[0] == 5.0 and np.isnan(m[1]) and m[2] == 3.0
    assert s[0] == 18.0 and np.isnan(s[1]) and s[2] == 9.0
    rng = np.random.default_rng(1236)
    y = rng.standard_normal((129, 777)).astype(np.float32)
    s, m, a, _ = oracle.rows_f32(y)
    np.testing.assert_allclose(s, y.astype(np.float64).sum(axis=1), rtol=1e-5, atol=1e-4)
    np.testing.assert_array_equal(m, y.max(axis=1))
    np.testing.assert_array_equal(a, y.argmax(axis=1).astype(np.uint32))
    idx, _ = oracle.arg_reduce(oracle.ARGMAX, y, oracle.FP32, [1])
    np.testing.assert_array_equal(a, idx.reshape(-1).astype(np.uint32))
