"""thor_scan_no_alloc (the scan entry point that allocates, compiles and loads nothing: temporary storage in the library's fixed
scratch block) against thor_scan through the C-ABI: same kernels, so every result is compared bit for bit, on two calls in a row
with the second one smaller than the first, plus its two refusals (kernels not loaded yet, request larger than the block)."""
from __future__ import annotations

import numpy as np
import pytest

from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, gpu_tensor
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import ScanOp

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def both(stream, carrier, dtype, op, inclusive=True, reverse=False, segment_size=0, offsets=None):
    """(thor_scan result, thor_scan_no_alloc result, variant) on the same device input; the output of the second call starts
    from a different fill so that a call that wrote nothing cannot pass."""
    x = copy_numpy_to_gpu(carrier, stream, dtype)
    arg = op in (ScanOp.arg_min, ScanOp.arg_max)
    out_dtype = DataType.uint32 if arg else dtype
    off = copy_numpy_to_gpu(np.asarray(offsets, np.uint32), stream, DataType.uint32) if offsets is not None else None
    want_t = gpu_tensor(list(carrier.shape), out_dtype)
    got_t = gpu_tensor(list(carrier.shape), out_dtype)
    got_t.memset_async(0x5A, stream)
    ph.scan(x, want_t, stream, op, inclusive, reverse, segment_size=segment_size, segment_offsets=off)
    variant = ph.scan(x, got_t, stream, op, inclusive, reverse, segment_size=segment_size, segment_offsets=off, no_alloc=True)
    return copy_gpu_to_numpy(want_t, stream), copy_gpu_to_numpy(got_t, stream), variant


def test_two_calls_in_a_row_second_smaller_match_the_allocating_entry_point(stream):
    rng = np.random.default_rng(7)
    # flat sums long enough for several chunks (the totals they publish to each other live in the scratch block), then a shorter one
    for n in (3_000_001, 70_003):
        x = rng.integers(0, 1 << 20, n, dtype=np.uint32)
        want, got, variant = both(stream, x, DataType.uint32, ScanOp.sum)
        assert "published_totals" in variant, variant
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(got, np.cumsum(x, dtype=np.uint32))
    for n in (1_500_007, 40_001):
        x = rng.standard_normal(n).astype(np.float32)
        want, got, _ = both(stream, x, DataType.fp32, ScanOp.sum, inclusive=False, reverse=True)
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_offset_segments_use_the_head_bitmap_in_the_block(stream):
    rng = np.random.default_rng(8)
    # the bitmap of the longer call must not leak into the shorter one: different partitions, second one smaller
    for n, segments in ((2_000_003, 5000), (300_001, 37)):
        cuts = np.sort(rng.integers(0, n, segments - 1))
        offsets = np.concatenate([[0], cuts, [n]])
        x = rng.standard_normal(n).astype(np.float32)
        want, got, variant = both(stream, x, DataType.fp32, ScanOp.max, offsets=offsets)
        assert variant.startswith("segments"), variant
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
        want, got, _ = both(stream, x, DataType.fp32, ScanOp.arg_min, offsets=offsets)
        np.testing.assert_array_equal(got, want)


def test_rows_longer_than_a_chunk(stream):
    rng = np.random.default_rng(9)
    for shape in ((7, 100_000), (3, 20_000)):
        x = rng.integers(0, 1000, shape, dtype=np.uint32)
        want, got, _ = both(stream, x, DataType.uint32, ScanOp.sum, segment_size=shape[1])
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(got, np.cumsum(x, axis=1, dtype=np.uint32))


def test_refuses_requests_whose_kernels_are_not_loaded(stream):
    n = 1_234_577  # a size no other test scans, so its kernels cannot be in the cache
    x = gpu_tensor([n], DataType.fp16)
    out = gpu_tensor([n], DataType.fp16)
    with pytest.raises(Exception, match="not loaded"):
        ph.scan(x, out, stream, ScanOp.min, inclusive=False, reverse=True, no_alloc=True)
    x.memset_async(0, stream)
    ph.scan(x, out, stream, ScanOp.min, inclusive=False, reverse=True)           # loads them
    ph.scan(x, out, stream, ScanOp.min, inclusive=False, reverse=True, no_alloc=True)
    stream.synchronize()


def test_refuses_requests_larger_than_the_block(stream):
    n = 1 << 26  # one head bit per element = 8 MiB of bitmap, twice the block
    x = gpu_tensor([n], DataType.uint32)
    out = gpu_tensor([n], DataType.uint32)
    off = copy_numpy_to_gpu(np.array([0, n // 2, n], np.uint32), stream, DataType.uint32)
    with pytest.raises(Exception, match="fixed scratch block"):
        ph.scan(x, out, stream, ScanOp.sum, segment_offsets=off, no_alloc=True)


def test_a_wait_that_gives_up_still_returns_complete_results(stream, monkeypatch):
    """This entry point has no temporary storage of the caller's to look into afterwards, so nothing could report a wait
    between blocks that gave up: such a wait works the totals it lacks out of the input instead.  Forced here with a bound of
    zero polls (a kernel of its own, loaded by the allocating call first)."""
    monkeypatch.setenv("THOR_SCAN_WAIT_LIMIT", "0")
    rng = np.random.default_rng(10)
    x = rng.integers(0, 1 << 20, 900_001, dtype=np.uint32)
    want, got, variant = both(stream, x, DataType.uint32, ScanOp.sum)
    assert "published_totals" in variant, variant
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got, np.cumsum(x, dtype=np.uint32))
