"""The oracle's select-flagged and top-k restatements against the reference's literal test vectors
(test/Utilities/TensorOperations/CubDevicePrimitivesTest.cpp:664-1003) and against what fixes them independently: NumPy's
sort of the key values, a brute-force rank count on small inputs, and a plain loop for the compaction."""
from __future__ import annotations

import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "selection_kats.json")) as f:
    KATS = json.load(f)
CODE = {"uint8": oracle.UINT8, "int8": oracle.INT8, "uint16": oracle.UINT16, "int16": oracle.INT16, "uint32": oracle.UINT32, "int32": oracle.INT32,
        "fp16": oracle.FP16, "bf16": oracle.BF16, "fp32": oracle.FP32}


def carriers(values, name):
    code = CODE[name]
    if name in ("fp16", "bf16"):
        return oracle.convert(np.array(values, np.float32), oracle.FP32, code)
    return np.array(values, oracle.CARRIER[code])


def as_values(carrier, name):
    if name in ("fp16", "bf16"):
        return oracle.convert(np.ascontiguousarray(carrier), CODE[name], oracle.FP32).astype(np.float64)
    return carrier.astype(np.float64)


@pytest.mark.parametrize("case", KATS["select"], ids=lambda c: f"{c['dtype']}-{c['num_items']}")
def test_select_reference_vectors(case):
    values = carriers(case["values"], case["dtype"])[:case["num_items"]]
    kept, count = oracle.select_flagged(values, np.array(case["flags"], np.uint8)[:case["num_items"]])
    assert count == len(case["expected"])
    np.testing.assert_array_equal(as_values(kept, case["dtype"]), np.array(case["expected"], np.float64))


@pytest.mark.parametrize("case", KATS["topk"] + KATS["segmented_topk"],
                         ids=lambda c: f"{c['dtype']}-k{c['k']}-{'largest' if c['largest'] else 'smallest'}-{c.get('segments', 0)}")
def test_top_k_reference_vectors(case):
    keys = carriers(case["keys"], case["dtype"])
    chosen, positions, _ = oracle.top_k(keys, case["k"], case["largest"], CODE[case["dtype"]], case.get("segment_size", 0))
    np.testing.assert_array_equal(as_values(chosen.reshape(-1), case["dtype"]), np.array(case["expected"], np.float64))
    if "values" in case:
        np.testing.assert_array_equal(np.array(case["values"])[positions.reshape(-1)], np.array(case["expected_values"]))


def test_select_matches_a_plain_loop():
    rng = np.random.default_rng(5)
    values = rng.integers(0, 1 << 32, 1000, dtype=np.uint64).astype(np.uint32)
    flags = (rng.random(1000) < 0.3).astype(np.uint8) * rng.integers(1, 255, 1000).astype(np.uint8)
    kept, count = oracle.select_flagged(values, flags)
    expected = [int(v) for v, f in zip(values, flags) if f]
    assert count == len(expected) and kept.tolist() == expected


@pytest.mark.parametrize("name", ["fp32", "fp16", "bf16", "int8", "int16", "int32", "uint8", "uint16", "uint32"])
def test_key_order_is_the_order_of_the_values(name):
    rng = np.random.default_rng(11)
    code = CODE[name]
    if name.startswith("fp") or name == "bf16":
        keys = carriers(np.concatenate([rng.standard_normal(500) * 50, [np.inf, -np.inf, 1e-30, -1e-30]]).astype(np.float32), name)
    else:
        info = np.iinfo(oracle.CARRIER[code])
        keys = rng.integers(info.min, int(info.max) + 1, 500).astype(oracle.CARRIER[code])
    image = oracle.key_order_image(keys, code)
    values = as_values(keys, name)
    by_image = values[np.argsort(image, kind="stable")]
    np.testing.assert_array_equal(by_image, np.sort(values))
    # equal images only for equal bit patterns
    assert len(np.unique(image)) == len(np.unique(keys.view(np.uint8).reshape(keys.size, -1), axis=0))


def test_float_specials_order_like_a_radix_sort():
    keys = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, -np.nan, 1.0, -1.0], np.float32)
    keys[5] = np.frombuffer(np.uint32(0xffc00000).tobytes(), np.float32)[0]
    image = oracle.key_order_image(keys, oracle.FP32)
    order = [int(i) for i in np.argsort(image)]
    assert order == [5, 3, 7, 1, 0, 6, 2, 4]  # -nan, -inf, -1, -0, +0, 1, +inf, +nan


@pytest.mark.parametrize("largest", [True, False])
def test_top_k_is_the_k_best_by_rank_count(largest):
    rng = np.random.default_rng(3)
    keys = rng.integers(0, 40, 200).astype(np.uint32)  # many ties
    for k in (1, 7, 50, 199, 200, 300):
        chosen, positions, threshold = oracle.top_k(keys, k, largest, oracle.UINT32)
        take = min(k, 200)
        assert chosen.shape == (1, take) and len(set(positions.reshape(-1).tolist())) == take
        np.testing.assert_array_equal(keys[positions.reshape(-1)], chosen.reshape(-1))
        # every key strictly better than the k-th is in the answer, nothing worse than it is
        better = keys > threshold[0] if largest else keys < threshold[0]
        assert set(np.nonzero(better)[0].tolist()) <= set(positions.reshape(-1).tolist())
        worst = chosen.min() if largest else chosen.max()
        assert worst == threshold[0] and better.sum() < take <= (better | (keys == threshold[0])).sum()


def test_top_k_of_rows_is_top_k_of_each_row():
    rng = np.random.default_rng(9)
    keys = rng.standard_normal((6, 33)).astype(np.float32)
    chosen, positions, _ = oracle.top_k(keys, 5, True, oracle.FP32, segment_size=33)
    for r in range(6):
        np.testing.assert_array_equal(chosen[r], np.sort(keys[r])[::-1][:5])
        np.testing.assert_array_equal(keys.reshape(-1)[positions[r]], chosen[r])
