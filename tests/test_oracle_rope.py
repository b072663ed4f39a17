"""The oracle's rotary position embedding against known answers worked out independently in double precision
(tests/golden/rope_kats.json, written by make_rope_kats.py), against what a rotation guarantees, and against the equivalences
the reference's own tests assert (test/Utilities/Expression/ExpressionConvenienceOpsTest.cpp:3503-3668)."""
import json
import os

import numpy as np
import pytest

import oracle

KINDS = {"none": oracle.ROPE_NONE, "linear": oracle.ROPE_LINEAR, "dynamic_ntk": oracle.ROPE_DYNAMIC_NTK, "yarn": oracle.ROPE_YARN,
         "longrope": oracle.ROPE_LONGROPE, "llama3": oracle.ROPE_LLAMA3}
with open(os.path.join(os.path.dirname(__file__), "golden", "rope_kats.json")) as f:
    CASES = json.load(f)["cases"]


def oracle_kwargs(case):
    kw = dict(case["options"])
    kw["scaling_kind"] = KINDS[kw.get("scaling_kind", "none")]
    kw["position_ids"] = case["position_ids"]
    kw["effective_sequence_length"] = case["effective_sequence_length"]
    return kw


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_known_answers(case):
    x = np.array(case["x"], np.float32).reshape(case["shape"])
    got = oracle.rope(x, oracle.FP32, **oracle_kwargs(case))
    want = np.array(case["expected"], np.float64).reshape(case["shape"])
    # fp32 angles and products against the double-precision answer: a few units in the last place of values up to ~4
    np.testing.assert_allclose(got, want, rtol=0, atol=4e-6)


def test_known_answers_cover_every_scaling_kind_and_layout():
    kinds = {c["options"].get("scaling_kind", "none") for c in CASES}
    assert kinds == set(KINDS)
    assert any(c["options"].get("interleaved") for c in CASES) and any(c["options"].get("inverse") for c in CASES)
    assert any(c["position_ids"] for c in CASES) and any(c["effective_sequence_length"] for c in CASES)
    assert any(c["options"].get("head_dim_axis", 3) < c["options"].get("sequence_axis", 2) for c in CASES)


def test_closed_form_first_pair():
    """Pair 0 has frequency base^0 = 1: the unit vector (1, 0) at position p becomes (cos p, sin p)."""
    x = np.zeros((1, 1, 6, 8), np.float32)
    x[..., 0] = 1.0
    y = oracle.rope(x, oracle.FP32)
    p = np.arange(6, dtype=np.float64)
    np.testing.assert_allclose(y[0, 0, :, 0], np.cos(p), atol=1e-6)
    np.testing.assert_allclose(y[0, 0, :, 4], np.sin(p), atol=1e-6)
    assert np.all(y[..., [1, 2, 3, 5, 6, 7]] == 0)
    yi = oracle.rope(x, oracle.FP32, interleaved=True)
    np.testing.assert_allclose(yi[0, 0, :, 1], np.sin(p), atol=1e-6)


@pytest.mark.parametrize("interleaved", [False, True])
def test_rotation_properties(interleaved):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 11, 16)).astype(np.float32)
    kw = dict(rotary_dim=12, interleaved=interleaved, position_offset=2)
    y = oracle.rope(x, oracle.FP32, **kw)
    # the tail of the head dimension is untouched, position 0 would be the identity
    assert np.array_equal(y[..., 12:], x[..., 12:])
    y0 = oracle.rope(x, oracle.FP32, rotary_dim=12, interleaved=interleaved)
    assert np.array_equal(y0[:, :, 0], x[:, :, 0])
    # each pair keeps its length
    first = np.arange(0, 12, 2) if interleaved else np.arange(6)
    second = first + 1 if interleaved else first + 6
    np.testing.assert_allclose(y[..., first] ** 2 + y[..., second] ** 2, x[..., first] ** 2 + x[..., second] ** 2, rtol=2e-6)
    # the inverse undoes it, and turning by p then q is turning by p + q
    np.testing.assert_allclose(oracle.rope(y, oracle.FP32, inverse=True, **kw), x, atol=2e-6)
    twice = oracle.rope(oracle.rope(x, oracle.FP32, rotary_dim=12, interleaved=interleaved, position_offset=3), oracle.FP32, **kw)
    # (offsets add only where positions are offsets alone: compare at sequence coordinate 0, whose positions are 3 then 2)
    once = oracle.rope(x, oracle.FP32, rotary_dim=12, interleaved=interleaved, position_offset=5)
    np.testing.assert_allclose(twice[:, :, 0], once[:, :, 0], atol=3e-6)
    # linear in the values; the attention factor scales the rotated part only
    np.testing.assert_allclose(oracle.rope(2 * x, oracle.FP32, **kw), 2 * y, atol=1e-6)
    scaled = oracle.rope(x, oracle.FP32, attention_factor=1.5, **kw)
    np.testing.assert_allclose(scaled[..., :12], np.float32(1.5) * y[..., :12], atol=2e-6)
    assert np.array_equal(scaled[..., 12:], x[..., 12:])


def test_interleaved_is_the_split_layout_permuted():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((1, 2, 5, 8)).astype(np.float32)
    split_order = np.concatenate([np.arange(0, 8, 2), np.arange(1, 8, 2)])  # interleaved coordinate of each split coordinate
    y_split = oracle.rope(np.ascontiguousarray(x[..., split_order]), oracle.FP32)
    y_inter = oracle.rope(x, oracle.FP32, interleaved=True)
    assert np.array_equal(y_inter[..., split_order], y_split)


def test_equivalences_the_reference_tests_assert():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((1, 2, 8, 8)).astype(np.float32)
    # Dynamic NTK whose effective length stays within the original maximum is the unscaled rotation; the physical extent (8 > 4)
    # is not (ExpressionConvenienceOpsTest.cpp:3503-3549)
    ntk = dict(rotary_dim=4, scaling_kind=oracle.ROPE_DYNAMIC_NTK, scaling_factor=2.0, original_max_position_embeddings=4)
    plain = oracle.rope(x, oracle.FP32, rotary_dim=4)
    assert np.array_equal(oracle.rope(x, oracle.FP32, effective_sequence_length=3, **ntk), plain)
    assert not np.array_equal(oracle.rope(x, oracle.FP32, **ntk), plain)
    # LongRoPE picks the short factors for a short effective length (:3551-3607)
    long_kw = dict(rotary_dim=4, scaling_kind=oracle.ROPE_LONGROPE, scaling_factor=1.0, original_max_position_embeddings=4,
                   long_rope_short_factors=[1.0, 1.0], long_rope_long_factors=[2.0, 2.0])
    assert np.array_equal(oracle.rope(x, oracle.FP32, effective_sequence_length=3, **long_kw), plain)
    assert not np.array_equal(oracle.rope(x, oracle.FP32, **long_kw), plain)
    # explicit absolute positions equal the scalar offset they spell out (:3627-3668)
    ids = np.arange(8) + 5
    assert np.array_equal(oracle.rope(x, oracle.FP32, rotary_dim=4, position_ids=ids), oracle.rope(x, oracle.FP32, rotary_dim=4, position_offset=5))


def test_storage_types_round_once():
    rng = np.random.default_rng(8)
    x = rng.standard_normal((1, 2, 5, 8)).astype(np.float32)
    for dt in (oracle.FP16, oracle.BF16):
        stored = oracle.from_f32(x.reshape(-1), dt).reshape(x.shape)
        want = oracle.from_f32(oracle.rope(oracle.to_f32(stored.reshape(-1), dt).reshape(x.shape), oracle.FP32).reshape(-1), dt).reshape(x.shape)
        assert np.array_equal(oracle.rope(stored, dt), want)
        assert oracle.rope(stored, dt, out_dtype=oracle.FP32).dtype == np.float32
