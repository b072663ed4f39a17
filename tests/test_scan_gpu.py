"""Prefix scans through the C-ABI (thor_scan over cubDeviceScan / cubDeviceSegmentedUniformScan / cubDeviceSegmentedScan and their
arg forms) against the oracle: bit-exact for UINT32, for min / max and for arg scans in every dtype; float sums and products
within a tolerance that covers the order of the additions (the reference's library fixes no order either) and, for 16-bit
floats, the reference's rounding of every partial result."""
from __future__ import annotations

import json
import os

import numpy as np
import pytest

import oracle
from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, gpu_tensor, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import ScanOp

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "scan_kats.json")) as f:
    KATS = json.load(f)["cases"]
ORACLE_OP = {ScanOp.sum: oracle.SCAN_SUM, ScanOp.min: oracle.SCAN_MIN, ScanOp.max: oracle.SCAN_MAX, ScanOp.product: oracle.SCAN_PRODUCT,
             ScanOp.arg_min: oracle.SCAN_ARGMIN, ScanOp.arg_max: oracle.SCAN_ARGMAX}


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def run_scan(carrier, dtype, stream, op, inclusive, reverse, segment_size=0, offsets=None, offsets_dtype=DataType.uint32):
    x = copy_numpy_to_gpu(carrier, stream, dtype)
    arg = op in (ScanOp.arg_min, ScanOp.arg_max)
    out = gpu_tensor(list(carrier.shape), DataType.uint32 if arg else dtype)
    off = None
    if offsets is not None:
        off = copy_numpy_to_gpu(np.asarray(offsets, np.uint32 if offsets_dtype == DataType.uint32 else np.uint64), stream, offsets_dtype)
    variant = ph.scan(x, out, stream, op, inclusive, reverse, segment_size=segment_size, segment_offsets=off)
    return copy_gpu_to_numpy(out, stream), variant


@pytest.mark.parametrize("case", KATS, ids=lambda c: f"{c['kind']}-{c['dtype']}-{c['op']}-{'incl' if c['inclusive'] else 'excl'}{'-rev' if c['reverse'] else ''}")
def test_reference_vectors(stream, case):
    dtype = DataType.uint32 if case["dtype"] == "uint32" else DataType.fp32
    values = np.array(case["values"], np.uint32 if dtype == DataType.uint32 else np.float32)
    kwargs = {"offsets": case["offsets"]} if case["kind"] == "segments" else {"segment_size": values.shape[-1]}
    got, _ = run_scan(values, dtype, stream, ScanOp[case["op"]], case["inclusive"], case["reverse"], **kwargs)
    np.testing.assert_array_equal(got.astype(np.float64), np.array(case["expected"], np.float64))


def check(got, carrier, dtype, op, inclusive, reverse, **segments):
    code = int(dtype)
    expected = oracle.scan(carrier, ORACLE_OP[op], inclusive, reverse, dtype=code, **segments)
    exact = dtype == DataType.uint32 or op != ScanOp.sum  # the product cases are built from exact factors
    if exact:
        np.testing.assert_array_equal(got, expected)
        return
    # float sums: compare against the fp32 prefix sums rounded once to the element type, with the error that another order of
    # the additions (and the last rounding) may leave: a few units in the last place of the sum of magnitudes
    values = from_storage(carrier, dtype).astype(np.float64).reshape(-1)
    gotf = from_storage(got, dtype).astype(np.float64).reshape(-1)
    reference = from_storage(oracle.scan(values.astype(np.float32), ORACLE_OP[op], inclusive, reverse, dtype=oracle.FP32, **segments), DataType.fp32)
    reference = from_storage(to_storage(reference, dtype), dtype)  # what a store of the fp32 prefix holds (overflow to inf included)
    unit = {DataType.fp32: 2.0 ** -24, DataType.fp16: 2.0 ** -11, DataType.bf16: 2.0 ** -8}[dtype]
    magnitude = from_storage(oracle.scan(np.abs(values).astype(np.float32), oracle.SCAN_SUM, True, reverse, dtype=oracle.FP32, **segments), DataType.fp32)
    slack = magnitude.astype(np.float64).reshape(-1) * unit * 2 + (64 * 2.0 ** -24) * magnitude.astype(np.float64).reshape(-1) + 1e-30
    assert np.all(np.abs(gotf - reference.astype(np.float64).reshape(-1)) <= slack)

SHAPES = [("rows", (300, 64)), ("rows", (5, 4099)), ("rows", (3, 70000)), ("rows", (2048, 3)), ("flat", (1, 1 << 20))]


SCAN_OPS = [ScanOp.sum, ScanOp.min, ScanOp.max, ScanOp.product, ScanOp.arg_min, ScanOp.arg_max]
SCAN_DTYPES = [DataType.uint32, DataType.fp32, DataType.fp16, DataType.bf16]
SCAN_MODES = [(True, False), (False, False), (True, True), (False, True)]  # (inclusive, reverse)
# Shape (which chunking the planner picks), dtype and operation (the arithmetic): every pair of the three meets - a shape takes
# every other (dtype, operation) pair, the halves alternating from shape to shape, so each (dtype, operation) pair runs on two or
# three shapes (every generated kernel is compiled on the spot, about half a second each: the full product took twice the time).
# Mode and direction are switches of the same code: each case takes one of their four combinations, turning.
ROWS_AND_FLAT = [(k, s, d, o, *SCAN_MODES[(i + j + m) % 4]) for i, (k, s) in enumerate(SHAPES) for j, d in enumerate(SCAN_DTYPES) for m, o in enumerate(SCAN_OPS)
                 if (i + j + m) % 2 == 0]


@pytest.mark.parametrize("kind,shape,dtype,op,inclusive,reverse", ROWS_AND_FLAT,
                         ids=[f"{k}{s}-{d.name}-{o.name}-{'incl' if i else 'excl'}{'-rev' if r else ''}" for k, s, d, o, i, r in ROWS_AND_FLAT])
def test_rows_and_flat_scans(stream, kind, shape, dtype, op, inclusive, reverse):
    rng = np.random.default_rng(41)
    n = shape[0] * shape[1]
    if dtype == DataType.uint32:
        carrier = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32) if op != ScanOp.product else rng.integers(1, 4, n).astype(np.uint32)
    elif op == ScanOp.product:
        # signed powers of two whose running exponent stays within +-6: every partial product, in any order, is exact in every
        # float dtype, so the products must agree bit for bit
        walk = np.clip(np.cumsum(rng.integers(-1, 2, n)), -6, 6)
        steps = np.diff(np.concatenate([[0], walk]))
        carrier = to_storage((np.exp2(steps) * rng.choice([1.0, -1.0], n)).astype(np.float32), dtype)
    else:
        carrier = to_storage((np.round(rng.standard_normal(n) * 8) / 8).astype(np.float32), dtype)  # many equal values: ties matter
    carrier = carrier.reshape(shape)
    segment_size = shape[1] if kind == "rows" else 0
    got, variant = run_scan(carrier, dtype, stream, op, inclusive, reverse, segment_size=segment_size)
    check(got, carrier, dtype, op, inclusive, reverse, segment_size=segment_size)
    if kind == "rows" and shape[1] <= 1000:
        assert "passes=scan)" in variant or "passes=scan," in variant  # rows that fit a block need no carries


# every (dtype, operation) with one of the four (inclusive, reverse) combinations and one of the two offset widths, both turning
OFFSET_SEGMENTED = [(d, o, *SCAN_MODES[(j + m) % 4], (DataType.uint32, DataType.uint64)[(m + j) % 2])
                    for j, d in enumerate([DataType.uint32, DataType.fp32, DataType.bf16])
                    for m, o in enumerate([ScanOp.sum, ScanOp.min, ScanOp.max, ScanOp.arg_min, ScanOp.arg_max])]


@pytest.mark.parametrize("dtype,op,inclusive,reverse,offsets_dtype", OFFSET_SEGMENTED,
                         ids=[f"{d.name}-{o.name}-{'incl' if i else 'excl'}{'-rev' if r else ''}-off_{w.name}" for d, o, i, r, w in OFFSET_SEGMENTED])
def test_offset_segmented_scans(stream, dtype, op, inclusive, reverse, offsets_dtype):
    rng = np.random.default_rng(43)
    n = 60000
    cuts = np.sort(rng.integers(0, n, 400))
    cuts[100:110] = cuts[100]  # empty segments
    cuts[200:203] = [cuts[200], cuts[200] + 1, cuts[200] + 2]  # and segments of one element
    offsets = np.concatenate([[0], np.sort(cuts), [n - 37]])  # the last 37 elements belong to no segment
    if dtype == DataType.uint32:
        carrier = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    else:
        carrier = to_storage((np.round(rng.standard_normal(n) * 8) / 8).astype(np.float32), dtype)
    got, variant = run_scan(carrier, dtype, stream, op, inclusive, reverse, offsets=offsets, offsets_dtype=offsets_dtype)
    active = int(offsets[-1])
    expected = oracle.scan(carrier, ORACLE_OP[op], inclusive, reverse, offsets=offsets, dtype=int(dtype))
    if dtype == DataType.uint32 or op != ScanOp.sum:
        np.testing.assert_array_equal(got[:active], expected[:active])
    else:
        check(got[:active], carrier[:active], dtype, op, inclusive, reverse, offsets=offsets)
    assert "segments(" in variant and "published_totals" in variant


def test_full_size_properties(stream):
    """2^26 fp32 elements: the last element of an inclusive sum scan of ones counts them; the exclusive scan is the inclusive
    one shifted; a reverse scan of the reversed input is the reversed forward scan; rows scanned independently."""
    n = 1 << 26
    host = np.ones(n, np.uint32)
    x = copy_numpy_to_gpu(host, stream, DataType.uint32)
    inclusive, exclusive = gpu_tensor([n], DataType.uint32), gpu_tensor([n], DataType.uint32)
    ph.scan(x, inclusive, stream, ScanOp.sum, True)
    ph.scan(x, exclusive, stream, ScanOp.sum, False)
    got_inclusive, got_exclusive = copy_gpu_to_numpy(inclusive, stream), copy_gpu_to_numpy(exclusive, stream)
    np.testing.assert_array_equal(got_inclusive, np.arange(1, n + 1, dtype=np.uint32))
    np.testing.assert_array_equal(got_exclusive, np.arange(0, n, dtype=np.uint32))
    rng = np.random.default_rng(47)
    values = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    forward, backward = gpu_tensor([n], DataType.uint32), gpu_tensor([n], DataType.uint32)
    ph.scan(copy_numpy_to_gpu(values, stream, DataType.uint32), forward, stream, ScanOp.max, True)
    ph.scan(copy_numpy_to_gpu(values[::-1].copy(), stream, DataType.uint32), backward, stream, ScanOp.max, True, reverse=True)
    np.testing.assert_array_equal(copy_gpu_to_numpy(forward, stream), np.maximum.accumulate(values))
    np.testing.assert_array_equal(copy_gpu_to_numpy(backward, stream)[::-1], np.maximum.accumulate(values))
    rows = gpu_tensor([n], DataType.uint32)
    ph.scan(copy_numpy_to_gpu(values, stream, DataType.uint32), rows, stream, ScanOp.sum, True, segment_size=1 << 13)
    np.testing.assert_array_equal(copy_gpu_to_numpy(rows, stream).reshape(-1, 1 << 13),
                                  (np.cumsum(values.reshape(-1, 1 << 13).astype(np.uint64), axis=1) & 0xFFFFFFFF).astype(np.uint32))


def test_validation(stream):
    x = copy_numpy_to_gpu(np.zeros(64, np.float32), stream, DataType.fp32)
    with pytest.raises(ValueError, match="Unsupported CUB scan dtype"):
        ph.scan(copy_numpy_to_gpu(np.zeros(64, np.int32), stream, DataType.int32), gpu_tensor([64], DataType.int32), stream)
    with pytest.raises(ValueError, match="dtypes must match"):
        ph.scan(x, gpu_tensor([64], DataType.fp16), stream)
    with pytest.raises(ValueError, match="arg scan output must be UINT32"):
        ph.scan(x, gpu_tensor([64], DataType.fp32), stream, ScanOp.arg_max)
    with pytest.raises(ValueError, match="num_segments \\* segment_size"):
        ph.scan(x, gpu_tensor([64], DataType.fp32), stream, segment_size=7)
    with pytest.raises(ValueError, match="offsets must be UINT32 or UINT64"):
        ph.scan(x, gpu_tensor([64], DataType.fp32), stream, segment_offsets=copy_numpy_to_gpu(np.zeros(3, np.float32), stream, DataType.fp32))


PUBLISHED = [  # (n, segments, dtype, op, reverse): every level of totals, every class of operation, both directions
    (16_800_001, 0, DataType.uint32, ScanOp.sum, False), (16_800_001, 0, DataType.fp32, ScanOp.sum, True), (16_800_001, 3, DataType.fp32, ScanOp.min, False),
    (16_800_001, 3, DataType.bf16, ScanOp.arg_max, True), (1_000_000, 2000, DataType.uint32, ScanOp.sum, True),
    (1_000_000, 2000, DataType.fp32, ScanOp.sum, False), (1_000_000, 2000, DataType.bf16, ScanOp.arg_max, False), (1_000_000, 0, DataType.fp32, ScanOp.min, True)]


@pytest.mark.parametrize("n,segments,dtype,op,reverse", PUBLISHED, ids=[f"{n}-{s}seg-{d.name}-{o.name}{'-rev' if r else ''}" for n, s, d, o, r in PUBLISHED])
def test_published_totals_agree_with_separate_passes(stream, monkeypatch, n, segments, dtype, op, reverse):
    """Chunks that read what precedes them from the totals other blocks publish (one launch over the data) against the same
    scan with totals and carries computed by launches of their own: the same bits for exact operations; float sums agree with
    the oracle within the bound of another order of additions and are the same bits from run to run.  The odd length keeps
    one element per lane and round, so 16.8 million elements are 4102 chunks: all three levels of published totals are read."""
    rng = np.random.default_rng(47)
    if dtype == DataType.uint32:
        carrier = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    else:
        carrier = to_storage((np.round(rng.standard_normal(n) * 8) / 8).astype(np.float32), dtype)
    offsets = None
    if segments:
        cuts = np.sort(rng.integers(0, n, segments - 1))
        offsets = np.concatenate([[0], cuts, [n]])
    got, variant = run_scan(carrier, dtype, stream, op, True, reverse, offsets=offsets)
    assert "published_totals" in variant, variant
    again, _ = run_scan(carrier, dtype, stream, op, True, reverse, offsets=offsets)
    np.testing.assert_array_equal(again.view(np.uint8), got.view(np.uint8))
    monkeypatch.setenv("THOR_SCAN_PASSES", "3")
    separate, variant = run_scan(carrier, dtype, stream, op, True, reverse, offsets=offsets)
    assert "totals+carries+scan" in variant, variant
    if dtype == DataType.uint32 or op != ScanOp.sum:
        np.testing.assert_array_equal(got, separate)
        kwargs = {"offsets": offsets} if segments else {}
        np.testing.assert_array_equal(got, oracle.scan(carrier, ORACLE_OP[op], True, reverse, dtype=int(dtype), **kwargs))
    elif segments:
        check(got, carrier, dtype, op, True, reverse, offsets=offsets)
        check(separate, carrier, dtype, op, True, reverse, offsets=offsets)
    else:
        check(got, carrier, dtype, op, True, reverse)
        check(separate, carrier, dtype, op, True, reverse)


@pytest.mark.parametrize("dtype,op,inclusive,reverse", [(DataType.uint32, ScanOp.sum, True, False), (DataType.fp32, ScanOp.max, False, True),
                                                        (DataType.bf16, ScanOp.arg_min, True, False)], ids=["u32-sum", "fp32-max-excl-rev", "bf16-argmin"])
def test_rows_longer_than_a_chunk_at_a_size_that_takes_the_large_blocks(stream, dtype, op, inclusive, reverse):
    """672 rows of 50 257 elements (33.8 million): every row spans several chunks of the 1 024-thread blocks, heads fall inside
    vectors, and a chunk reads what precedes it in its row from totals published by other blocks, two levels deep."""
    rng = np.random.default_rng(53)
    rows, length = 672, 50257
    if dtype == DataType.uint32:
        carrier = rng.integers(0, 1 << 32, rows * length, dtype=np.uint64).astype(np.uint32)
    else:
        carrier = to_storage((np.round(rng.standard_normal(rows * length) * 8) / 8).astype(np.float32), dtype)
    carrier = carrier.reshape(rows, length)
    got, variant = run_scan(carrier, dtype, stream, op, inclusive, reverse, segment_size=length)
    assert "threads=1024" in variant and "published_totals" in variant, variant
    check(got, carrier, dtype, op, inclusive, reverse, segment_size=length)


def test_a_wait_that_gives_up_works_its_totals_out_again(stream, monkeypatch):
    """Waits between blocks are bounded so that every wavefront has an exit.  With the bound forced to zero polls every chunk
    that needs the total of an earlier one gives up at once and works that total out from the input, in the order its owner
    would have: flat, ragged and float-sum scans return the bits of the ordinary run, through thor_scan and through the Scan
    stage of a stamped Expression, and thor_scan counts the waits that took the way out."""
    rng = np.random.default_rng(59)
    ones = np.ones(1 << 22, np.uint32)
    noisy = rng.standard_normal(1_300_003).astype(np.float32)      # odd length: single elements, 318 chunks, five groups
    cuts = np.sort(rng.integers(0, noisy.size, 99))
    offsets = np.concatenate([[0], cuts, [noisy.size]])
    rows = rng.integers(0, 1 << 32, (3, 70_001), dtype=np.uint64).astype(np.uint32)
    ordinary = {
        "flat": run_scan(ones, DataType.uint32, stream, ScanOp.sum, True, False),
        "float": run_scan(noisy, DataType.fp32, stream, ScanOp.sum, False, True),
        "ragged": run_scan(noisy, DataType.fp32, stream, ScanOp.arg_max, True, False, offsets=offsets),
    }
    for got, variant in ordinary.values():
        assert "published_totals" in variant, variant
    np.testing.assert_array_equal(ordinary["flat"][0], np.arange(1, ones.size + 1, dtype=np.uint32))
    before = ph.scan_waits_recovered()
    monkeypatch.setenv("THOR_SCAN_WAIT_LIMIT", "0")
    recovered = {
        "flat": run_scan(ones, DataType.uint32, stream, ScanOp.sum, True, False),
        "float": run_scan(noisy, DataType.fp32, stream, ScanOp.sum, False, True),
        "ragged": run_scan(noisy, DataType.fp32, stream, ScanOp.arg_max, True, False, offsets=offsets),
    }
    assert ph.scan_waits_recovered() >= before + 3 * 100  # nearly every chunk waits for an earlier one of its group
    for name, (got, variant) in recovered.items():
        assert "published_totals" in variant, variant
        np.testing.assert_array_equal(got.view(np.uint32), ordinary[name][0].view(np.uint32), err_msg=name)
    # the Scan stage of a stamped Expression: rows longer than a chunk, so chunks inside a row read earlier totals
    x = copy_numpy_to_gpu(rows, stream, DataType.uint32)
    plan = ph.Expression.compile(ph.Expression.input("x").scan(ScanOp.sum), 0).stamp({"x": x}, stream)
    assert plan.stage_kind_names() == ["Scan"]
    plan.run()
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output(), stream), np.cumsum(rows, axis=1, dtype=np.uint32))
