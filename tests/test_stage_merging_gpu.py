"""Stored values that other values of the same shape read: one kernel keeps the producer in registers and stores it too, when
what is stored is what was computed; the plan with one stage per level gives the same bits."""
from __future__ import annotations

import os

import numpy as np
import pytest

from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def stamp_and_run(outputs, tensors, stream, staged):
    if staged:
        os.environ["THOR_DISABLE_STAGE_FUSION"] = "1"
    try:
        plan = ex.compile(ex.outputs(outputs), device_num=0).stamp(tensors, stream)
    finally:
        os.environ.pop("THOR_DISABLE_STAGE_FUSION", None)
    plan.run()
    return plan


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
def test_chain_of_named_outputs_runs_as_one_kernel(stream, dtype):
    rng = np.random.default_rng(3)
    a, b = (to_storage(rng.uniform(-1, 1, (257, 33)).astype(np.float32), dtype) for _ in range(2))
    tensors = {"a": copy_numpy_to_gpu(a, stream, dtype), "b": copy_numpy_to_gpu(b, stream, dtype)}
    x, y = ex.input("a"), ex.input("b")
    product = x * y
    shifted = product.exp() + x
    outputs = {"product": product, "shifted": shifted, "ratio": shifted / (product * product + 1.0)}
    merged = stamp_and_run(outputs, tensors, stream, staged=False)
    staged = stamp_and_run(outputs, tensors, stream, staged=True)
    assert merged.stage_kind_names() == ["FusedKernel"]
    assert staged.stage_kind_names() == ["FusedKernel"] * 3
    for name in outputs:
        np.testing.assert_array_equal(copy_gpu_to_numpy(merged.output(name), stream), copy_gpu_to_numpy(staged.output(name), stream))
    af, bf = from_storage(a, dtype).astype(np.float64), from_storage(b, dtype).astype(np.float64)
    tolerance = 1e-6 if dtype == DataType.fp32 else 2e-2
    np.testing.assert_allclose(from_storage(copy_gpu_to_numpy(merged.output("ratio"), stream), dtype), (np.exp(af * bf) + af) / ((af * bf) ** 2 + 1),
                               rtol=tolerance, atol=tolerance)


def test_values_stored_narrower_than_computed_or_read_through_views_keep_their_stage(stream):
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, (64, 48)).astype(np.float32)
    tensors = {"a": copy_numpy_to_gpu(a, stream, DataType.fp32)}
    x = ex.input("a")
    narrow = (x * 3.0).with_output_dtype(DataType.fp16)  # computed in fp32, stored as fp16: readers see the rounded value
    plan = stamp_and_run({"narrow": narrow, "reader": narrow.cast(DataType.fp32) + 1.0}, tensors, stream, staged=False)
    stored = from_storage(copy_gpu_to_numpy(plan.output("narrow"), stream), DataType.fp16)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("reader"), stream), stored + np.float32(1))
    doubled = x * 2.0
    viewed = stamp_and_run({"doubled": doubled, "folded": doubled.reshape([48, 64]).exp()}, tensors, stream, staged=False)
    assert viewed.stage_kind_names() == ["FusedKernel", "FusedKernel"]  # different shape: a second kernel reads the stored tensor
    np.testing.assert_allclose(copy_gpu_to_numpy(viewed.output("folded"), stream), np.exp((a * 2).reshape(48, 64)), rtol=2e-6)
