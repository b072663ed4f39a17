"""Select-flagged and top-k through the C-ABI (thor_select_flagged / thor_topk over cubDeviceSelectFlagged, cubDeviceTopKKeys / Pairs
and cubDeviceSegmentedTopKKeys / Pairs) against the oracle.  The compaction is compared bit for bit, in order.  Top-k output is
unordered in the reference and which of several equal keys is taken is not fixed, so the keys are compared bit for bit after
sorting, and the values of pairs by what they point at: every returned (key, value) pair must be a pair of the input and no input
position may be returned twice."""
from __future__ import annotations

import json
import os

import numpy as np
import pytest

import oracle
from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, gpu_tensor, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType, numpy_carrier

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "selection_kats.json")) as f:
    KATS = json.load(f)
KEY_DTYPES = [DataType.uint8, DataType.int8, DataType.uint16, DataType.int16, DataType.uint32, DataType.int32, DataType.fp16, DataType.bf16,
              DataType.fp32]
FLOATS = (DataType.fp16, DataType.bf16, DataType.fp32)


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def carriers(values, dtype):
    if dtype in FLOATS:
        return to_storage(np.array(values, np.float32), dtype)
    return np.array(values, numpy_carrier(dtype))


def random_keys(rng, n, dtype, distinct_levels=None):
    if dtype in FLOATS:
        values = rng.standard_normal(n).astype(np.float32) * 100
        if distinct_levels:
            values = np.round(values / 100 * distinct_levels)
        return to_storage(values, dtype)
    info = np.iinfo(numpy_carrier(dtype))
    low, high = (info.min, int(info.max) + 1) if not distinct_levels else (max(info.min, -distinct_levels), min(int(info.max) + 1, distinct_levels))
    return rng.integers(low, high, n).astype(numpy_carrier(dtype))


def bits_of(carrier):
    return np.ascontiguousarray(carrier).view({1: np.uint8, 2: np.uint16, 4: np.uint32}[carrier.dtype.itemsize])


def sorted_by_order(carrier, dtype, largest):
    image = oracle.key_order_image(carrier, int(dtype))
    order = np.argsort(-image if largest else image, kind="stable")
    return bits_of(carrier.reshape(-1))[order]


# ---- select-flagged ----------------------------------------------------------------------------------------------------------------
def run_select(values, flags, dtype, flag_dtype, stream, num_items=None, count_before=77):
    n = values.size if num_items is None else num_items
    x = copy_numpy_to_gpu(values, stream, dtype)
    f = copy_numpy_to_gpu(flags, stream, flag_dtype)
    out = copy_numpy_to_gpu(np.zeros(max(values.size, 1), numpy_carrier(dtype)), stream, dtype)
    count = copy_numpy_to_gpu(np.array([count_before], np.uint32), stream, DataType.uint32)
    variant = ph.select_flagged(x, f, out, count, stream, num_items=n)
    return copy_gpu_to_numpy(out, stream), int(copy_gpu_to_numpy(count, stream)[0]), variant


@pytest.mark.parametrize("case", KATS["select"], ids=lambda c: f"{c['dtype']}-{c['num_items']}")
def test_select_reference_vectors(stream, case):
    dtype, flag_dtype = DataType[case["dtype"]], DataType[case["flag_dtype"]]
    values = carriers(case["values"], dtype)
    got, count, _ = run_select(values, np.array(case["flags"], np.uint8), dtype, flag_dtype, stream, case["num_items"])
    assert count == len(case["expected"])
    np.testing.assert_array_equal(bits_of(got[:count]), bits_of(carriers(case["expected"], dtype)))


# elements are copied as raw words: one dtype of each width meets every length, the other dtypes two lengths each
SELECT_LENGTHS = [1, 63, 4095, 4096, 4097, 1_000_003]
SELECT_CASES = [(d, n) for d in (DataType.uint8, DataType.bf16, DataType.fp32) for n in SELECT_LENGTHS]
SELECT_CASES += [(d, SELECT_LENGTHS[(2 * i + j) % 6]) for i, d in enumerate(d for d in KEY_DTYPES if d not in (DataType.uint8, DataType.bf16, DataType.fp32))
                 for j in (0, 3)]


@pytest.mark.parametrize("dtype,n", SELECT_CASES, ids=[f"{d.name}-{n}" for d, n in SELECT_CASES])
def test_select_keeps_the_flagged_elements_in_order(stream, dtype, n):
    rng = np.random.default_rng(n * 31 + int(dtype))
    values = random_keys(rng, n, dtype)
    flags = ((rng.random(n) < 0.37) * rng.integers(1, 256, n)).astype(np.uint8)
    got, count, variant = run_select(values, flags, dtype, DataType.uint8, stream)
    expected, expected_count = oracle.select_flagged(values, flags)
    assert count == expected_count and "select-flagged" in variant
    np.testing.assert_array_equal(bits_of(got[:count]), bits_of(expected))
    np.testing.assert_array_equal(bits_of(got[count:]), 0)  # nothing is written past the selected elements


@pytest.mark.parametrize("density", [0.0, 1.0, 0.001, 0.999])
def test_select_at_extreme_densities_with_boolean_flags(stream, density):
    n = 300_000
    rng = np.random.default_rng(int(density * 1000) + 1)
    values = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    flags = (rng.random(n) < density).astype(np.uint8)
    got, count, _ = run_select(values, flags, DataType.uint32, DataType.boolean, stream)
    expected, expected_count = oracle.select_flagged(values, flags)
    assert count == expected_count
    np.testing.assert_array_equal(got[:count], expected)


def test_select_over_a_prefix_of_larger_tensors(stream):
    rng = np.random.default_rng(8)
    values = rng.standard_normal(10_000).astype(np.float32)
    flags = (rng.random(10_000) < 0.5).astype(np.uint8)
    got, count, _ = run_select(values, flags, DataType.fp32, DataType.uint8, stream, num_items=6_001)
    expected, expected_count = oracle.select_flagged(values[:6_001], flags[:6_001])
    assert count == expected_count
    np.testing.assert_array_equal(got[:count], expected)


def test_select_full_size_partition_round_trip(stream):
    """2^26 elements: the flagged elements and the unflagged ones together are the input, each part in input order."""
    n = 1 << 26
    rng = np.random.default_rng(26)
    values = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    flags = (rng.random(n) < 0.5).astype(np.uint8)
    kept, kept_count, _ = run_select(values, flags, DataType.uint32, DataType.uint8, stream)
    dropped, dropped_count, _ = run_select(values, 1 - flags, DataType.uint32, DataType.uint8, stream)
    assert kept_count == int(flags.sum()) and kept_count + dropped_count == n
    merged = np.empty(n, np.uint32)
    merged[flags != 0] = kept[:kept_count]
    merged[flags == 0] = dropped[:dropped_count]
    np.testing.assert_array_equal(merged, values)


def test_select_rejects_what_the_reference_rejects(stream):
    x = gpu_tensor([4], DataType.uint32)
    flags = gpu_tensor([4], DataType.uint8)
    count = gpu_tensor([1], DataType.uint32)
    with pytest.raises(ValueError, match="input/output dtypes must match"):
        ph.select_flagged(x, flags, gpu_tensor([4], DataType.fp32), count, stream)
    with pytest.raises(ValueError, match="Unsupported CUB select flag dtype"):
        ph.select_flagged(x, gpu_tensor([4], DataType.fp32), gpu_tensor([4], DataType.uint32), count, stream)
    with pytest.raises(ValueError, match="num_selected_out must have dtype uint32"):
        ph.select_flagged(x, flags, gpu_tensor([4], DataType.uint32), gpu_tensor([1], DataType.fp32), stream)
    with pytest.raises(ValueError, match="output has fewer elements than num_items"):
        ph.select_flagged(x, flags, gpu_tensor([3], DataType.uint32), count, stream)
    with pytest.raises(ValueError, match="Unsupported CUB select value dtype"):
        ph.select_flagged(gpu_tensor([4], DataType.fp8_e4m3), flags, gpu_tensor([4], DataType.fp8_e4m3), count, stream)


# ---- top-k -------------------------------------------------------------------------------------------------------------------------
def run_top_k(keys, dtype, k, largest, stream, pairs=False, segment_size=None, values=None):
    flat = keys.reshape(-1)
    run = segment_size if segment_size else flat.size
    segments = flat.size // run if run else 0
    take = min(k, run)
    x = copy_numpy_to_gpu(flat, stream, dtype)
    out = copy_numpy_to_gpu(np.zeros(max(segments * take, 1), numpy_carrier(dtype)), stream, dtype)
    values_in = values_out = None
    if pairs:
        values = np.arange(flat.size, dtype=np.uint32) if values is None else np.asarray(values, np.uint32)
        values_in = copy_numpy_to_gpu(values, stream, DataType.uint32)
        values_out = copy_numpy_to_gpu(np.full(max(segments * take, 1), 0xffffffff, np.uint32), stream, DataType.uint32)
    variant = ph.top_k(x, out, k, stream, largest=largest, values_in=values_in, values_out=values_out,
                       **({"segment_size": segment_size, "num_segments": segments} if segment_size else {"num_items": flat.size}))
    got = copy_gpu_to_numpy(out, stream)[:segments * take].reshape(segments, take)
    got_values = copy_gpu_to_numpy(values_out, stream)[:segments * take].reshape(segments, take) if pairs else None
    return got, got_values, variant


def check_top_k(keys, dtype, k, largest, got, got_values, segment_size=None):
    flat = keys.reshape(-1)
    expected, _, _ = oracle.top_k(flat, k, largest, int(dtype), segment_size or 0)
    assert got.shape == expected.shape
    for row in range(expected.shape[0]):
        np.testing.assert_array_equal(sorted_by_order(got[row], dtype, largest), bits_of(expected[row]))
    if got_values is not None:
        run = segment_size or flat.size
        for row in range(expected.shape[0]):
            positions = got_values[row].astype(np.int64)
            assert len(np.unique(positions)) == positions.size
            assert positions.min() >= row * run and positions.max() < (row + 1) * run
            np.testing.assert_array_equal(bits_of(flat[positions]), bits_of(got[row]))


@pytest.mark.parametrize("case", KATS["topk"] + KATS["segmented_topk"],
                         ids=lambda c: f"{c['dtype']}-k{c['k']}-{'largest' if c['largest'] else 'smallest'}-{c.get('segments', 0)}")
def test_top_k_reference_vectors(stream, case):
    dtype = DataType[case["dtype"]]
    keys = carriers(case["keys"], dtype)
    segment_size = case.get("segment_size")
    got, got_values, _ = run_top_k(keys, dtype, case["k"], case["largest"], stream, pairs="values" in case, segment_size=segment_size,
                                   values=case.get("values"))
    expected = carriers(case["expected"], dtype).reshape(got.shape)
    for row in range(got.shape[0]):
        np.testing.assert_array_equal(sorted_by_order(got[row], dtype, case["largest"]), bits_of(expected[row]))
    if "values" in case:
        pairs = sorted(zip(bits_of(got.reshape(-1)).tolist(), got_values.reshape(-1).tolist()))
        assert pairs == sorted(zip(bits_of(expected.reshape(-1)).tolist(), case["expected_values"]))


# every key dtype meets every (n, k); the order alternates so that every dtype and every (n, k) sees both
TOPK_SIZES = [(1, 1), (257, 256), (2049, 2049), (100_003, 1), (100_003, 1000), (1_000_000, 65_537)]
TOPK_KEY_CASES = [(d, (i + j) % 2 == 0, n, k) for i, d in enumerate(KEY_DTYPES) for j, (n, k) in enumerate(TOPK_SIZES)]


@pytest.mark.parametrize("dtype,largest,n,k", TOPK_KEY_CASES, ids=[f"{d.name}-{'largest' if l else 'smallest'}-{n}-{k}" for d, l, n, k in TOPK_KEY_CASES])
def test_top_k_keys(stream, dtype, largest, n, k):
    rng = np.random.default_rng(n * 7 + k + int(dtype))
    keys = random_keys(rng, n, dtype)
    got, _, variant = run_top_k(keys, dtype, k, largest, stream)
    assert "radix-select" in variant
    check_top_k(keys, dtype, k, largest, got, None)


@pytest.mark.parametrize("dtype", [DataType.uint8, DataType.int16, DataType.fp16, DataType.fp32, DataType.uint32], ids=lambda d: d.name)
@pytest.mark.parametrize("largest", [True, False], ids=["largest", "smallest"])
def test_top_k_pairs_with_many_equal_keys(stream, dtype, largest):
    rng = np.random.default_rng(int(dtype) + 100)
    keys = random_keys(rng, 200_000, dtype, distinct_levels=20)
    for k in (1, 4_000, 150_000):
        got, got_values, _ = run_top_k(keys, dtype, k, largest, stream, pairs=True)
        check_top_k(keys, dtype, k, largest, got, got_values)


# the key kinds of two and four bytes (unsigned, signed, float), each with roomy lists and with lists that overflow, orders alternating
CANDIDATE_MODES = [("roomy", {}), ("short-list", {"THOR_TOPK_REGION": "1"}), ("short-second-list", {"THOR_TOPK_AMBIGUOUS": "2"}),
                   ("both-short", {"THOR_TOPK_REGION": "1", "THOR_TOPK_AMBIGUOUS": "2"})]
CANDIDATE_CASES = [(d, (i + j) % 2 == 0, CANDIDATE_MODES[j][0], CANDIDATE_MODES[j][1])
                   for i, d in enumerate([DataType.uint16, DataType.int32, DataType.bf16, DataType.fp32, DataType.fp16])
                   for j in ((0, 1, 2, 3) if d in (DataType.fp32, DataType.uint16) else ({DataType.int32: 3, DataType.bf16: 2, DataType.fp16: 0}[d],))]


@pytest.mark.parametrize("dtype,largest,mode,switches", CANDIDATE_CASES,
                         ids=[f"{d.name}-{'largest' if l else 'smallest'}-{m}" for d, l, m, _ in CANDIDATE_CASES])
def test_top_k_over_candidates(stream, monkeypatch, dtype, largest, mode, switches):
    """Long inputs list the keys above a floor taken from a sample (the keys that can still be part of the answer) during the one
    pass over the input and finish on that list; the switch asks for that on short inputs and large k too (down to no sample: a
    floor of zero).  A list that is too short makes the last launch walk the whole input, a second list (the keys of the
    bucket that holds the k-th) that is too short makes its last block walk the candidates again: every way must give the same answer."""
    monkeypatch.setenv("THOR_TOPK_CANDIDATES", "1")
    for name, value in switches.items():
        monkeypatch.setenv(name, value)
    rng = np.random.default_rng(int(dtype) * 3 + largest)
    sizes = ((100_003, 1000, None), (300_001, 4_000, 20), (300_001, 250_000, 20), (65_536, 65_536, None), (1 << 20, 300, None))
    turn = CANDIDATE_CASES.index((dtype, largest, mode, switches))  # three of the five sizes per case, turning (each size compiles six kernels)
    for index, (n, k, levels) in enumerate(sizes):
        if (index + turn) % 5 in (1, 3):
            continue
        keys = random_keys(rng, n, dtype, distinct_levels=levels)
        got, got_values, variant = run_top_k(keys, dtype, k, largest, stream, pairs=True)
        assert "candidates(" in variant and "launches3" in variant
        check_top_k(keys, dtype, k, largest, got, got_values)
        if index in (0, 4):  # the key-only kernels are the pair kernels without the positions: two of the five sizes
            got, _, _ = run_top_k(keys, dtype, k, largest, stream)
            check_top_k(keys, dtype, k, largest, got, None)


def test_top_k_with_fewer_than_k_keys_above_the_floor(stream):
    """Many keys equal to the k-th largest: the floor is that key, the list holds the few keys above it and the rest of the
    answer are keys equal to the floor, from positions noted during the pass (pairs) or written as copies of the key."""
    rng = np.random.default_rng(5)
    keys = np.maximum(rng.standard_normal(1 << 21).astype(np.float32), 0)  # half of them zero
    keys[rng.integers(0, keys.size, 1 << 19)] = np.float32(2.5)               # and about a quarter the same positive value
    for k, largest in ((700_000, True), (8_000, True), (100, False), (5_000, False)):
        for pairs in (True, False):
            if k * 256 > keys.size:
                continue
            got, got_values, variant = run_top_k(keys, DataType.fp32, k, largest, stream, pairs=pairs)
            assert "candidates(" in variant
            check_top_k(keys, DataType.fp32, k, largest, got, got_values if pairs else None)
    ints = rng.integers(0, 3, 1 << 20).astype(np.int32)  # three values: every k-th largest has a third of the input equal to it
    for k in (1, 4_000):
        got, got_values, _ = run_top_k(ints, DataType.int32, k, True, stream, pairs=True)
        check_top_k(ints, DataType.int32, k, True, got, got_values)


def test_top_k_long_inputs_use_candidates_by_default(stream):
    rng = np.random.default_rng(77)
    keys = rng.standard_normal((1 << 21) + 12).astype(np.float32)
    keys[rng.integers(0, keys.size, 50)] = np.float32(9.5)  # ties at the top
    for k in (1, 40, 64, 8_000, 70_000):
        got, got_values, variant = run_top_k(keys, DataType.fp32, k, True, stream, pairs=True)
        assert ("candidates(" in variant) == (k * 256 <= keys.size)  # a k beyond a 256th of the input reads it once per digit
        check_top_k(keys, DataType.fp32, k, True, got, got_values)
    sorted_keys = np.sort(keys)  # every candidate in one stretch of the input
    for largest in (True, False):
        got, got_values, _ = run_top_k(sorted_keys, DataType.fp32, 3_000, largest, stream, pairs=True)
        check_top_k(sorted_keys, DataType.fp32, 3_000, largest, got, got_values)


def test_top_k_of_equal_keys_and_k_beyond_the_input(stream):
    keys = np.full(10_000, 7, np.uint32)
    got, got_values, _ = run_top_k(keys, DataType.uint32, 99_999, True, stream, pairs=True)
    check_top_k(keys, DataType.uint32, 99_999, True, got, got_values)
    assert got.shape == (1, 10_000)


def test_top_k_float_specials(stream):
    """-0 below +0, infinities at the ends, NaNs beyond them by sign: the order of the key bits."""
    specials = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 1e-45, -1e-45], np.float32)
    negative_nan = np.frombuffer(np.uint32(0xffc00001).tobytes(), np.float32)
    rng = np.random.default_rng(4)
    keys = np.concatenate([specials, negative_nan, rng.standard_normal(5_000).astype(np.float32)])
    rng.shuffle(keys)
    for largest in (True, False):
        for k in (1, 2, 3, 5, 2_505):
            got, _, _ = run_top_k(keys, DataType.fp32, k, largest, stream)
            check_top_k(keys, DataType.fp32, k, largest, got, None)


def test_top_k_zero_k_leaves_the_output_alone(stream):
    keys = copy_numpy_to_gpu(np.arange(8, dtype=np.uint32), stream, DataType.uint32)
    out = copy_numpy_to_gpu(np.full(4, 99, np.uint32), stream, DataType.uint32)
    assert ph.top_k(keys, out, 0, stream) == ""
    np.testing.assert_array_equal(copy_gpu_to_numpy(out, stream), 99)


# Rows a wavefront can hold (at most 64 keys per lane) take the kernel with one wavefront per row: a bit-by-bit search over the
# keys in registers, or - when at most 64 keys are wanted and every lane holds two groups of vectors - over the few keys at or
# above a floor taken from the groups' maxima ("floor-candidates"); longer rows take one block per row.  Every key dtype meets five of the seven shapes (every shape at least six of the nine dtypes), the
# order alternating: rows of two keys, rows no vector divides, almost all keys wanted, rows of one vector per lane, full rows of
# 4096, the longest rows, many short rows.
ROW_SHAPES = [(1, 2, 1), (33, 257, 256), (100, 1000, 10), (37, 4096, 64), (6, 8192, 8191), (3000, 64, 8), (50, 3000, 3)]
ROW_CASES = [(d, (i + j) % 2 == 0, *shape) for i, d in enumerate(KEY_DTYPES) for j, shape in enumerate(ROW_SHAPES) if (i + j) % 7 not in (2, 5)]


def row_kernel_form(dtype, segment_size, k):
    """What the variant text of a row top-k says about the kernel the planner must have chosen."""
    vec = 16 // np.dtype(numpy_carrier(dtype)).itemsize
    vectors_per_lane = -(-segment_size // (64 * vec))
    if vectors_per_lane * vec > 64:
        return "block-per-row"
    floor = k <= 64 and vectors_per_lane % 2 == 0 and segment_size >= 32 * vec * vectors_per_lane and vectors_per_lane * vec > 16
    return "wavefront-per-row" + (" floor-candidates" if floor else "")


@pytest.mark.parametrize("dtype,largest,segments,segment_size,k", ROW_CASES,
                         ids=[f"{d.name}-{'largest' if l else 'smallest'}-{s}x{n}-k{k}" for d, l, s, n, k in ROW_CASES])
def test_top_k_of_rows(stream, dtype, largest, segments, segment_size, k):
    rng = np.random.default_rng(segments * 13 + segment_size + k + int(dtype))
    keys = random_keys(rng, segments * segment_size, dtype)
    got, got_values, variant = run_top_k(keys, dtype, k, largest, stream, pairs=True, segment_size=segment_size)
    form = row_kernel_form(dtype, segment_size, k)
    assert "row top-k" in variant and form.split()[0] in variant and ("floor-candidates" in variant) == ("floor-candidates" in form), variant
    check_top_k(keys, dtype, k, largest, got, got_values, segment_size=segment_size)


@pytest.mark.parametrize("dtype,segment_size,k,levels", [(DataType.bf16, 300, 100, 6), (DataType.bf16, 4096, 64, 6), (DataType.fp32, 2048, 33, 3),
                                                         (DataType.uint8, 4096, 5, None), (DataType.int16, 1536, 64, 40)],
                         ids=["bf16-300-k100", "bf16-4096-k64", "fp32-2048-k33", "uint8-4096-k5", "int16-1536-k64"])
def test_top_k_of_rows_keys_only_with_ties(stream, dtype, segment_size, k, levels):
    """Few distinct keys: the threshold key is shared by many, and with a floor most of a row lies at or above it - more
    candidates than a wavefront's part of LDS holds, so those rows finish with the search over all keys.  One row is a single
    repeated key, one holds the extremes of the order."""
    rng = np.random.default_rng(77)
    rows = 96
    keys = random_keys(rng, rows * segment_size, dtype, distinct_levels=levels).reshape(rows, segment_size)
    keys[3] = keys[3, 0]
    if dtype in FLOATS:
        keys[5, :7] = to_storage(np.array([np.inf, -np.inf, np.nan, 0.0, -0.0, np.inf, np.nan], np.float32), dtype)
    for largest in (True, False):
        got, _, variant = run_top_k(keys, dtype, k, largest, stream, segment_size=segment_size)
        assert "wavefront-per-row" in variant, variant
        check_top_k(keys, dtype, k, largest, got, None, segment_size=segment_size)


def test_both_row_kernels_agree(stream, monkeypatch):
    """The switch forces one block per row on rows a wavefront could hold: the same keys, sorted, from both kernels."""
    rng = np.random.default_rng(78)
    keys = random_keys(rng, 64 * 4096, DataType.fp16).reshape(64, 4096)
    by_wavefront, values_w, variant = run_top_k(keys, DataType.fp16, 64, True, stream, pairs=True, segment_size=4096)
    assert "wavefront-per-row" in variant and "floor-candidates" in variant, variant
    monkeypatch.setenv("THOR_TOPK_ROW_KERNEL", "block")
    by_block, values_b, variant = run_top_k(keys, DataType.fp16, 64, True, stream, pairs=True, segment_size=4096)
    assert "block-per-row" in variant, variant
    for row in range(64):
        np.testing.assert_array_equal(sorted_by_order(by_wavefront[row], DataType.fp16, True), sorted_by_order(by_block[row], DataType.fp16, True))
    check_top_k(keys, DataType.fp16, 64, True, by_wavefront, values_w, segment_size=4096)
    check_top_k(keys, DataType.fp16, 64, True, by_block, values_b, segment_size=4096)


@pytest.mark.parametrize("dtype", [DataType.bf16, DataType.fp32, DataType.int16], ids=lambda d: d.name)
def test_rows_whose_candidates_crowd_one_lane(stream, dtype):
    """The wavefront-per-row kernel keeps the keys at or above its floor on lane-private stacks: 8 entries of every lane in
    registers as a rule, up to 16 with a wider search, beyond that the search over all of the row's registers.  Rows of 4 096
    keys in which one lane (lane l holds keys (64 j + l) * V .. + V of every j) owns 0, 10, 16, 17, 40 ... of the best keys."""
    rng = np.random.default_rng(int(dtype) + 500)
    vec = 16 // np.dtype(numpy_carrier(dtype)).itemsize
    crowds = [0, 10, 16, 17, 40, 12, 9, 64]
    if dtype in FLOATS:
        values = rng.standard_normal((len(crowds), 4096)).astype(np.float32) * 100
    else:
        values = rng.integers(-30000, 30000, (len(crowds), 4096)).astype(np.int32)
    for largest in (True, False):
        rows = values.copy()
        for row, crowd in enumerate(crowds):
            lane = 5 + row
            own = np.array([(64 * j + lane) * vec + e for j in range(4096 // (64 * vec)) for e in range(vec)])  # the lane's 64 positions
            order = np.argsort(rows[row])
            best = (order[::-1] if largest else order)[:crowd]  # swap the row's `crowd` best keys into that lane
            for target, source in zip(own[:crowd], best):
                rows[row, [target, source]] = rows[row, [source, target]]
        keys = to_storage(rows, dtype) if dtype in FLOATS else rows.astype(numpy_carrier(dtype))
        got, got_values, variant = run_top_k(keys, dtype, 64, largest, stream, pairs=True, segment_size=4096)
        assert "wavefront-per-row" in variant and "floor-candidates" in variant, variant
        check_top_k(keys, dtype, 64, largest, got, got_values, segment_size=4096)


def test_sorted_rows_whose_best_keys_all_sit_in_the_first_lane(stream):
    """2 763 ascending fp16 rows of 1 518 keys, the 5 smallest with their positions: every answer is in lane 0's first vector and
    takes output slots 0..4 in that order.  The slot of a key is the number of voting lanes below its own; computed from a mask
    `(1 << lane) - 1` this kernel once gave slots 1..5 for about 1 % of the rows, other rows on every run: the mask's 64-bit shift
    had its amount in the last vector register the wavefront owned (v63 of 64), which MI355X gets wrong one time in ten.  The
    count now comes from mbcnt.  Several runs, since the failure came and went."""
    rng = np.random.default_rng(11)
    segments, size, k = 2763, 1518, 5
    keys = to_storage(np.sort(rng.standard_normal((segments, size)).astype(np.float32), axis=1).reshape(-1), DataType.fp16)
    for _ in range(3):
        got, got_values, variant = run_top_k(keys, DataType.fp16, k, False, stream, pairs=True, segment_size=size)
        assert "wavefront-per-row" in variant, variant
        check_top_k(keys, DataType.fp16, k, False, got, got_values, segment_size=size)


def test_top_k_full_size_against_a_host_partition(stream):
    """2^26 fp32 keys, k = 2^16: the answer's smallest key is the k-th largest of the input and every key above it is present
    (checked with NumPy's partition, which shares nothing with the radix selection)."""
    n, k = 1 << 26, 1 << 16
    rng = np.random.default_rng(2026)
    keys = rng.standard_normal(n).astype(np.float32)
    got, got_values, _ = run_top_k(keys, DataType.fp32, k, True, stream, pairs=True)
    kth = np.partition(keys, n - k)[n - k]
    assert got.min() == kth
    assert int((keys > kth).sum()) == int((got > kth).sum())
    positions = got_values.reshape(-1).astype(np.int64)
    assert len(np.unique(positions)) == k
    np.testing.assert_array_equal(keys[positions], got.reshape(-1))
    np.testing.assert_array_equal(np.sort(got.reshape(-1)), np.sort(np.partition(keys, n - k)[n - k:]))


def test_top_k_rejects_what_the_reference_rejects(stream):
    keys = gpu_tensor([15], DataType.uint32)
    with pytest.raises(ValueError, match="key input/output dtypes must match"):
        ph.top_k(keys, gpu_tensor([2], DataType.fp32), 2, stream)
    with pytest.raises(ValueError, match="Unsupported CUB top-k key dtype"):
        ph.top_k(gpu_tensor([2], DataType.fp8_e4m3), gpu_tensor([1], DataType.fp8_e4m3), 1, stream)
    with pytest.raises(ValueError, match="Unsupported CUB top-k index value dtype"):
        ph.top_k(keys, gpu_tensor([2], DataType.uint32), 2, stream, values_in=gpu_tensor([15], DataType.fp32), values_out=gpu_tensor([2], DataType.fp32))
    with pytest.raises(ValueError, match="keys_out has fewer elements than num_items"):
        ph.top_k(keys, gpu_tensor([1], DataType.uint32), 2, stream)
    with pytest.raises(ValueError, match="requires k to be smaller than the fixed segment size"):
        ph.top_k(keys, gpu_tensor([15], DataType.uint32), 5, stream, segment_size=5, num_segments=3)
    with pytest.raises(ValueError, match="segment_size exceeds"):
        ph.top_k(gpu_tensor([8193 * 2], DataType.uint32), gpu_tensor([2], DataType.uint32), 1, stream, segment_size=8193, num_segments=2)
    with pytest.raises(ValueError, match="segment_size must be nonzero"):
        ph.top_k(keys, gpu_tensor([3], DataType.uint32), 1, stream, segment_size=0, num_segments=3)
    with pytest.raises(ValueError, match="Unsupported CUB segmented top-k key dtype"):
        ph.top_k(gpu_tensor([4], DataType.fp64), gpu_tensor([2], DataType.fp64), 1, stream, segment_size=2, num_segments=2)


def test_prepared_plans_share_one_temporary_storage_and_run_repeatedly(stream):
    """PreparedPlansCanShareOnePreallocatedWorkspace / PreparedPlanRejectsUndersizedWorkspace of the reference's tests
    (CubDevicePrimitivesTest.cpp:1787-1930), for the plans built here."""
    rng = np.random.default_rng(90)
    n = 300_000
    keys = rng.standard_normal(n).astype(np.float32)
    flags = (rng.random(n) < 0.25).astype(np.uint8)
    x = copy_numpy_to_gpu(keys, stream, DataType.fp32)
    f = copy_numpy_to_gpu(flags, stream, DataType.uint8)
    picked, count = gpu_tensor([n], DataType.fp32), gpu_tensor([1], DataType.uint32)
    best, best_at = gpu_tensor([1000], DataType.fp32), gpu_tensor([1000], DataType.uint32)
    positions = copy_numpy_to_gpu(np.arange(n, dtype=np.uint32), stream, DataType.uint32)
    select = ph.SelectionPlan.select_flagged(x, f, picked, count)
    top = ph.SelectionPlan.top_k(x, best, 1000, largest=False, values_in=positions, values_out=best_at)
    assert "select-flagged" in select.variant() and "smallest pairs" in top.variant()
    temp = gpu_tensor([max(select.temp_storage_bytes, top.temp_storage_bytes)], DataType.uint8)
    for _ in range(3):
        select.run(temp, x, f, picked, count, stream=stream)
        top.run(temp, x, best, positions, best_at, stream=stream)
        expected, expected_count = oracle.select_flagged(keys, flags)
        assert int(copy_gpu_to_numpy(count, stream)[0]) == expected_count
        np.testing.assert_array_equal(copy_gpu_to_numpy(picked, stream)[:expected_count], expected)
        check_top_k(keys, DataType.fp32, 1000, False, copy_gpu_to_numpy(best, stream).reshape(1, -1), copy_gpu_to_numpy(best_at, stream).reshape(1, -1))
    with pytest.raises(ValueError, match="temp_storage has fewer bytes"):
        select.run(gpu_tensor([16], DataType.uint8), x, f, picked, count, stream=stream)
    with pytest.raises(ValueError, match="plan is not compatible"):
        top.run(temp, copy_numpy_to_gpu(keys.astype(np.float16), stream, DataType.fp16), gpu_tensor([1000], DataType.fp16), positions, best_at, stream=stream)
