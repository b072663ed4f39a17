"""Plans with independent branches on helper streams (THOR_STAGE_OVERLAP=1: the reference's fork / join scheduling,
Utilities/Expression/StampedEquation.cpp:4115-4207 there) against the same plans on one stream (this build's default): the
values must not depend on the lanes, run after run, with inputs rewritten between runs."""
from __future__ import annotations

import os

import numpy as np
import pytest

from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def run_both_ways(plan, names, stream, refresh=None, rounds=3):
    results = {"serial": [], "forked": []}
    for r in range(rounds):
        if refresh is not None:
            refresh(r)
        for mode in ("serial", "forked"):
            if mode == "forked":
                os.environ["THOR_STAGE_OVERLAP"] = "1"
            try:
                plan.run()
            finally:
                os.environ.pop("THOR_STAGE_OVERLAP", None)
            results[mode].append({n: copy_gpu_to_numpy(plan.output(n), stream) for n in names})
    return results


def test_backward_of_min_and_max_branches(stream):
    rng = np.random.default_rng(3)
    x = ex.input("x")
    spread = (x.exp().reduce_max(axis=1) - (x * x).reduce_min(axis=1)).reduce_sum(axis=[0, 1])
    eq = ex.compile(spread, 0).compile_backward(["x"])
    values = rng.uniform(-2, 2, (500, 700)).astype(np.float32)
    tx = copy_numpy_to_gpu(values, stream, DataType.fp32)
    plan = eq.stamp({"x": tx}, stream)
    kinds = plan.stage_kind_names()
    assert kinds.count("ArgMinMax") == 2  # two independent branches

    def refresh(r):
        fresh = copy_numpy_to_gpu(np.roll(values, 13 * r, axis=1), stream, DataType.fp32)
        tx.copy_from_async(fresh, stream)  # queued on the caller's stream: helper lanes must wait for it

    got = run_both_ways(plan, ["x_grad"], stream, refresh)
    for r in range(3):
        np.testing.assert_array_equal(got["forked"][r]["x_grad"], got["serial"][r]["x_grad"])
        v = np.roll(values, 13 * r, axis=1).astype(np.float64)
        expected = np.zeros_like(v)
        rows = np.arange(v.shape[0])
        hi, lo = np.argmax(np.exp(v), axis=1), np.argmin(v * v, axis=1)
        expected[rows, hi] += np.exp(v[rows, hi])
        expected[rows, lo] -= 2 * v[rows, lo]
        np.testing.assert_allclose(got["forked"][r]["x_grad"], expected, rtol=2e-6, atol=1e-7)


def test_independent_reductions_of_different_inputs(stream):
    rng = np.random.default_rng(4)
    a = rng.integers(-8, 9, (300, 1000)).astype(np.float32)
    b = rng.integers(-8, 9, (300, 500)).astype(np.float32)
    c = rng.integers(-8, 9, (300, 64)).astype(np.float32)
    expr = ex.outputs({"mix": ex.input("a").reduce_sum(axis=1) * 2.0 + ex.input("b").reduce_max(axis=1) - ex.input("c").reduce_min(axis=1),
                       "norm": ex.input("c").abs().reduce_sum(axis=1)})
    plan = ex.compile(expr, 0).stamp({k: copy_numpy_to_gpu(v, stream, DataType.fp32) for k, v in (("a", a), ("b", b), ("c", c))}, stream)
    got = run_both_ways(plan, ["mix", "norm"], stream)
    want = a.sum(axis=1, keepdims=True) * 2 + b.max(axis=1, keepdims=True) - c.min(axis=1, keepdims=True)
    for r in range(3):
        for mode in ("serial", "forked"):
            np.testing.assert_array_equal(got[mode][r]["mix"], want)  # small integers: exact in any order
            np.testing.assert_array_equal(got[mode][r]["norm"], np.abs(c).sum(axis=1, keepdims=True))
