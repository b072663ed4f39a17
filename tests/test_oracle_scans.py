"""The scan oracle against the literal vectors of the reference's tests (tests/golden/scan_kats.json) and against NumPy's
accumulate routines, which fix the results for integers and for min / max in any dtype."""
from __future__ import annotations

import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
OPS = {"sum": oracle.SCAN_SUM, "min": oracle.SCAN_MIN, "max": oracle.SCAN_MAX, "product": oracle.SCAN_PRODUCT, "arg_min": oracle.SCAN_ARGMIN,
       "arg_max": oracle.SCAN_ARGMAX}
with open(os.path.join(HERE, "golden", "scan_kats.json")) as f:
    KATS = json.load(f)["cases"]


@pytest.mark.parametrize("case", KATS, ids=lambda c: f"{c['kind']}-{c['dtype']}-{c['op']}-{'incl' if c['inclusive'] else 'excl'}{'-rev' if c['reverse'] else ''}")
def test_scan_known_answers(case):
    dtype = oracle.UINT32 if case["dtype"] == "uint32" else oracle.FP32
    values = np.array(case["values"], np.uint32 if dtype == oracle.UINT32 else np.float32)
    kwargs = {"offsets": case["offsets"]} if case["kind"] == "segments" else {"segment_size": values.shape[-1]}
    got = oracle.scan(values, OPS[case["op"]], case["inclusive"], case["reverse"], dtype=dtype, **kwargs)
    expected = np.array(case["expected"], dtype=np.float64)
    np.testing.assert_array_equal(got.astype(np.float64), expected)


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("inclusive", [True, False])
def test_scan_matches_numpy_accumulate(inclusive, reverse):
    rng = np.random.default_rng(31)
    rows, length = 7, 53
    ints = rng.integers(0, 1 << 31, (rows, length)).astype(np.uint32)
    floats = np.round(rng.standard_normal((rows, length)) * 4) / 4
    flip = (lambda a: a[:, ::-1]) if reverse else (lambda a: a)

    def shifted(inclusive_result, identity):
        if inclusive:
            return inclusive_result
        out = np.empty_like(inclusive_result)
        out[:, 0] = identity
        out[:, 1:] = inclusive_result[:, :-1]
        return out

    got = oracle.scan(ints, oracle.SCAN_SUM, inclusive, reverse, segment_size=length, dtype=oracle.UINT32)
    np.testing.assert_array_equal(got, flip(shifted(np.cumsum(flip(ints).astype(np.uint64), axis=1) & 0xFFFFFFFF, 0)).astype(np.uint32))
    got = oracle.scan(ints, oracle.SCAN_PRODUCT, inclusive, reverse, segment_size=length, dtype=oracle.UINT32)
    wrapped = np.empty((rows, length), np.uint64)
    run = np.ones(rows, np.uint64)
    for j in range(length):
        run = (run * flip(ints)[:, j].astype(np.uint64)) & np.uint64(0xFFFFFFFF)
        wrapped[:, j] = run
    np.testing.assert_array_equal(got, flip(shifted(wrapped, 1)).astype(np.uint32))
    for dtype in (oracle.FP32, oracle.FP16, oracle.BF16):
        stored = oracle.from_f32(floats.astype(np.float32), dtype)
        as_f32 = oracle.to_f32(stored, dtype)
        got = oracle.to_f32(oracle.scan(stored, oracle.SCAN_MIN, inclusive, reverse, segment_size=length, dtype=dtype), dtype)
        np.testing.assert_array_equal(got, flip(shifted(np.minimum.accumulate(flip(as_f32), axis=1), np.inf)))
        got = oracle.to_f32(oracle.scan(stored, oracle.SCAN_MAX, inclusive, reverse, segment_size=length, dtype=dtype), dtype)
        np.testing.assert_array_equal(got, flip(shifted(np.maximum.accumulate(flip(as_f32), axis=1), -np.inf)))
        # arg scans name the first element that attains the running extreme: values gathered at the indices are the value scan
        if inclusive and not reverse:
            index = oracle.scan(stored, oracle.SCAN_ARGMAX, True, False, segment_size=length, dtype=dtype)
            np.testing.assert_array_equal(as_f32.reshape(-1)[index.reshape(-1)].reshape(rows, length), np.maximum.accumulate(as_f32, axis=1))
            assert np.all(np.diff(index.astype(np.int64), axis=1) >= 0)
    # halves that overflow to infinity or absorb small addends do so in the oracle as they do element by element
    halves = oracle.from_f32(np.full((1, 40), 3000.0, np.float32), oracle.FP16)
    got = oracle.to_f32(oracle.scan(halves, oracle.SCAN_SUM, True, False, segment_size=40, dtype=oracle.FP16), oracle.FP16)
    with np.errstate(over="ignore"):
        sequential = np.cumsum(np.full(40, 3000.0, np.float16), dtype=np.float16).astype(np.float32)  # NumPy rounds every partial sum too
    np.testing.assert_array_equal(got[0], sequential)
    assert np.isinf(got[0, -1]) and got[0, 10] != 33000.0


@pytest.mark.parametrize("dtype", [oracle.UINT32, oracle.FP32, oracle.FP16, oracle.BF16])
@pytest.mark.parametrize("op", list(OPS.values()))
def test_the_three_engines_perform_the_same_walk(op, dtype):
    rng = np.random.default_rng(37)
    n = 700
    offsets = np.concatenate([[0], np.sort(rng.integers(0, n, 12)), [n - 5]])
    offsets[5] = offsets[4]
    if dtype == oracle.UINT32:
        values = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    else:
        values = oracle.from_f32((np.round(rng.standard_normal(n) * 4) / 4).astype(np.float32), dtype)
    for inclusive in (True, False):
        for reverse in (False, True):
            for kwargs in ({"offsets": offsets}, {"segment_size": 70}, {}):
                slow = oracle.scan(values, op, inclusive, reverse, dtype=dtype, engine="python", **kwargs)
                quick = oracle.scan(values, op, inclusive, reverse, dtype=dtype, engine="numpy", **kwargs)
                compiled = oracle.scan(values, op, inclusive, reverse, dtype=dtype, engine="c", **kwargs)
                np.testing.assert_array_equal(slow, quick)
                np.testing.assert_array_equal(slow, compiled)


@pytest.mark.parametrize("dtype", [oracle.UINT32, oracle.FP32, oracle.FP16, oracle.BF16])
def test_products_and_sixteen_bit_sums_round_at_every_step(dtype):
    """The cases NumPy has no sequential routine for (UINT32 products, bf16 sums and products): the compiled walk against the
    Python loop on inputs where rounding at every step shows (sums that absorb small addends, products that lose bits)."""
    rng = np.random.default_rng(39)
    n = 500
    if dtype == oracle.UINT32:
        values = rng.integers(1, 1 << 16, n).astype(np.uint32)
    else:
        values = oracle.from_f32(rng.uniform(0.9, 1.1, n).astype(np.float32), dtype)
    for op in (oracle.SCAN_SUM, oracle.SCAN_PRODUCT):
        for kwargs in ({"segment_size": 125}, {}):
            slow = oracle.scan(values, op, True, False, dtype=dtype, engine="python", **kwargs)
            compiled = oracle.scan(values, op, True, False, dtype=dtype, engine="c", **kwargs)
            np.testing.assert_array_equal(slow, compiled)
    if dtype == oracle.BF16:  # 256 + 1 is not a bf16 value: a running bf16 sum of ones stops at 256, an fp32 sum rounded once would not
        ones = oracle.from_f32(np.ones(400, np.float32), dtype)
        got = oracle.to_f32(oracle.scan(ones, oracle.SCAN_SUM, True, False, dtype=dtype), dtype)
        assert got[255] == 256.0 and got[-1] == 256.0
