"""launchSegmentedBroadcast: per-segment values onto packed ragged rows (reference semantics:
Utilities/Expression/SegmentedBroadcastKernel.cu:82-104), against a numpy loop over the segments."""
from __future__ import annotations

import numpy as np
import pytest

from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, gpu_tensor, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def expected(values_f32, offsets, filler_storage, dtype, normalize):
    """Rows of segment b get values[b] (divided in fp32 by the length and rounded once); other rows keep the filler."""
    out = filler_storage.copy()
    for b in range(len(offsets) - 1):
        lo, hi = int(offsets[b]), int(offsets[b + 1])
        if hi <= lo:
            continue
        row = values_f32[b]
        if normalize:
            row = to_storage((row.astype(np.float32) / np.float32(hi - lo)).astype(np.float32), dtype)
        else:
            row = to_storage(row, dtype)
        out[lo:hi] = row
    return out


def partitions(rng, rows, segments):
    cuts = np.sort(rng.integers(0, rows + 1, segments - 1)) if segments > 1 else np.array([], dtype=np.int64)
    full = np.concatenate([[0], cuts, [rows]]).astype(np.int64)
    partial = full.copy()
    partial[-1] = max(int(partial[-2]), rows - rows // 7)  # rows after the last segment belong to nobody
    with_empty = full.copy()
    if segments > 4:
        with_empty[2:4] = with_empty[2]
    return [full, partial, np.sort(with_empty)]


CASES = [((5000,), 37), ((4096, 8), 19), ((777, 3, 5), 12), ((300, 1024), 7), ((100000, 2), 5000), ((70000, 3), 1), ((200000,), 90000), ((33, 4099), 9)]


# every shape in fp32 and in one narrower dtype (the four take turns down the list: each meets two shapes)
NARROW = (DataType.bf16, DataType.fp16, DataType.fp8_e4m3, DataType.fp8_e5m2)
BROADCAST_CASES = [(s, b, d) for i, (s, b) in enumerate(CASES) for d in (DataType.fp32, NARROW[i % 4])]


@pytest.mark.parametrize("shape,segments,dtype", BROADCAST_CASES, ids=[f"{s}-{b}-{d.name}" for s, b, d in BROADCAST_CASES])
def test_broadcast_matches_a_loop_over_segments(stream, shape, segments, dtype):
    rng = np.random.default_rng(len(shape) * 1000 + segments)
    per_segment_shape = (segments,) + shape[1:]
    values = to_storage(rng.standard_normal(per_segment_shape).astype(np.float32) * 8, dtype)
    values_f32 = from_storage(values, dtype)
    tv = copy_numpy_to_gpu(values, stream, dtype)
    for index, offsets in enumerate(partitions(rng, shape[0], segments)):
        for offsets_dtype in (DataType.uint32, DataType.uint64):
            carrier = offsets.astype(np.uint64 if offsets_dtype == DataType.uint64 else np.uint32)
            toff = copy_numpy_to_gpu(carrier, stream, offsets_dtype)
            for normalize in (False, True):
                if offsets_dtype == DataType.uint64 and not normalize:
                    continue  # the offsets' width only changes how the partition is read
                filler = to_storage(np.full(shape, 77.0, np.float32), dtype)
                out = copy_numpy_to_gpu(filler, stream, dtype)
                ph.segmented_broadcast(tv, toff, out, normalize, stream)
                got = copy_gpu_to_numpy(out, stream)
                want = expected(values_f32, offsets, filler, dtype, normalize)
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), f"partition {index} {offsets_dtype.name} normalize={normalize}"


def test_trailing_shapes_may_differ_and_contract_violations_raise(stream):
    values = copy_numpy_to_gpu(np.arange(8, dtype=np.float32).reshape(2, 4), stream, DataType.fp32)
    offsets = copy_numpy_to_gpu(np.array([0, 1, 3], np.uint32), stream, DataType.uint32)
    out = gpu_tensor([3, 2, 2], DataType.fp32)
    ph.segmented_broadcast(values, offsets, out, False, stream)
    np.testing.assert_array_equal(copy_gpu_to_numpy(out, stream).reshape(3, 4), np.array([[0, 1, 2, 3], [4, 5, 6, 7], [4, 5, 6, 7]], np.float32))
    with pytest.raises(RuntimeError, match="batch_size \\+ 1"):
        ph.segmented_broadcast(values, copy_numpy_to_gpu(np.array([0, 1, 2, 3], np.uint32), stream, DataType.uint32), out, False, stream)
    with pytest.raises(RuntimeError, match="dtypes must match"):
        ph.segmented_broadcast(values, offsets, gpu_tensor([3, 4], DataType.fp16), False, stream)
    with pytest.raises(RuntimeError, match="elements-per-value"):
        ph.segmented_broadcast(values, offsets, gpu_tensor([3, 5], DataType.fp32), False, stream)
    with pytest.raises(RuntimeError, match="UINT32 or UINT64"):
        ph.segmented_broadcast(values, copy_numpy_to_gpu(np.array([0, 1, 3], np.float32), stream, DataType.fp32), out, False, stream)
