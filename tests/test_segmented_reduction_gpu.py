"""Offset-segmented reductions (CubSegmentedReduction / CubSegmentedArgReduction) against the reference tests' literal vectors
(tests/golden/segmented_kats.json) and against per-segment numpy results on random ragged partitions."""
from __future__ import annotations

import json
import os

import numpy as np
import pytest

from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, gpu_tensor, gpu_to_f32, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "segmented_kats.json")
VALUE_OPS = {"Sum": ph.CubReductionOp.Sum, "Mean": ph.CubReductionOp.Mean, "Min": ph.CubReductionOp.Min, "Max": ph.CubReductionOp.Max}
ARG_OPS = {"ArgMin": ph.CubArgReductionOp.ArgMin, "ArgMax": ph.CubArgReductionOp.ArgMax}


def kats():
    with open(GOLDEN) as f:
        return json.load(f)


def floats(values):
    table = {None: np.nan, "inf": np.inf, "-inf": -np.inf}
    return np.array([table.get(v, v) if (v is None or isinstance(v, str)) else v for v in values], dtype=np.float32)


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def upload_offsets(values, stream, dtype=DataType.uint32):
    carrier = np.asarray(values, dtype=np.uint64 if dtype == DataType.uint64 else np.uint32)
    return copy_numpy_to_gpu(carrier, stream, dtype)


@pytest.mark.parametrize("case", kats()["value"], ids=lambda c: c["name"])
def test_value_known_answers(stream, case):
    x = copy_numpy_to_gpu(floats(case["input"]).reshape(case["shape"]), stream, DataType.fp32)
    offsets = upload_offsets(case["offsets"], stream, DataType.uint64 if case.get("offsets_dtype") == "uint64" else DataType.uint32)
    for name, op in VALUE_OPS.items():
        if name not in case:
            continue
        stamped = ph.CubSegmentedReduction(op, DataType.fp32).stamp(x, offsets, stream)
        assert stamped.get_path() == ph.CubReductionPath.OffsetSegmented
        stamped.run()
        out = stamped.get_output_tensor()
        assert out.get_dimensions() == [len(case["offsets"]) - 1] + case["shape"][1:]
        np.testing.assert_allclose(gpu_to_f32(out, stream).reshape(-1), floats(case[name]), rtol=1e-6, err_msg=name)


@pytest.mark.parametrize("case", kats()["arg"], ids=lambda c: c["name"])
@pytest.mark.parametrize("index_dtype", [DataType.uint64, DataType.uint32], ids=lambda d: d.name)
@pytest.mark.parametrize("offsets_dtype", [DataType.uint32, DataType.uint64], ids=lambda d: "off_" + d.name)
def test_arg_known_answers(stream, case, index_dtype, offsets_dtype):
    x = copy_numpy_to_gpu(floats(case["input"]).reshape(case["shape"]), stream, DataType.fp32)
    offsets = upload_offsets(case["offsets"], stream, offsets_dtype)
    sentinel = np.iinfo(np.uint64 if index_dtype == DataType.uint64 else np.uint32).max
    for name, op in ARG_OPS.items():
        if name not in case:
            continue
        stamped = ph.CubSegmentedArgReduction(op, index_dtype).stamp(x, offsets, stream)
        stamped.run()
        got = copy_gpu_to_numpy(stamped.get_index_output_tensor(), stream).reshape(-1)
        want = [sentinel if v == "max" else v for v in case[name]]
        assert got.tolist() == want, name


def segment_reference(x64, offsets, op):
    """float64 per-segment results, [B, D...]."""
    out = []
    for b in range(len(offsets) - 1):
        rows = x64[offsets[b]:offsets[b + 1]]
        if rows.shape[0] == 0:
            empty = {"Sum": 0.0, "Mean": 0.0, "Min": np.inf, "Max": -np.inf}[op]
            out.append(np.full(x64.shape[1:], empty))
        else:
            out.append({"Sum": rows.sum(axis=0), "Mean": rows.mean(axis=0), "Min": rows.min(axis=0), "Max": rows.max(axis=0)}[op])
    return np.stack(out)


def ragged_offsets(rng, rows, segments):
    cuts = np.sort(rng.integers(0, rows + 1, segments - 1))
    offsets = np.concatenate([[0], cuts, [rng.integers(cuts[-1] if segments > 1 else 0, rows + 1)]])
    offsets[3:5] = offsets[3]  # a few empty segments
    return np.sort(offsets).astype(np.int64)


SHAPES = [((5000,), 37), ((4096, 8), 19), ((777, 3, 5), 12), ((300, 1024), 7), ((100000, 2), 5), ((64, 4099), 9), ((200000,), 1)]


# every shape in fp32 and in one narrower dtype (bf16, fp16 and fp8 take turns down the list)
RAGGED_CASES = [(s, b, d) for i, (s, b) in enumerate(SHAPES) for d in (DataType.fp32, (DataType.bf16, DataType.fp16, DataType.fp8_e4m3)[i % 3])]


@pytest.mark.parametrize("shape,segments,dtype", RAGGED_CASES, ids=[f"{s}-{b}-{d.name}" for s, b, d in RAGGED_CASES])
def test_random_ragged_partitions_against_numpy(stream, shape, segments, dtype):
    rng = np.random.default_rng(hash((shape, segments)) % 2**32)
    x = to_storage(rng.standard_normal(shape).astype(np.float32), dtype)
    xf = from_storage(x, dtype).astype(np.float64)
    offsets = ragged_offsets(rng, shape[0], segments) if segments > 1 else np.array([0, shape[0]])
    tx = copy_numpy_to_gpu(x, stream, dtype)
    toff = upload_offsets(offsets, stream)
    lengths = np.diff(offsets).reshape([-1] + [1] * (len(shape) - 1))
    for name, op in VALUE_OPS.items():
        stamped = ph.CubSegmentedReduction(op, DataType.fp32).stamp(tx, toff, stream)
        stamped.run()
        got = gpu_to_f32(stamped.get_output_tensor(), stream).astype(np.float64)
        want = segment_reference(xf, offsets, name)
        assert got.shape == want.shape
        if name in ("Min", "Max"):
            np.testing.assert_array_equal(got, want, err_msg=f"{name} {stamped.get_kernel_variant()}")
        else:
            absolute = segment_reference(np.abs(xf), offsets, "Sum") / (np.maximum(lengths, 1) if name == "Mean" else 1)
            assert np.all(np.abs(got - want) <= 1e-5 * absolute + 1e-30), f"{name} {stamped.get_kernel_variant()}"
    trailing = int(np.prod(shape[1:])) if len(shape) > 1 else 1
    flat = xf.reshape(shape[0], trailing)
    for name, op in ARG_OPS.items():
        stamped = ph.CubSegmentedArgReduction(op).stamp(tx, toff, stream)
        stamped.run()
        got = copy_gpu_to_numpy(stamped.get_index_output_tensor(), stream).reshape(len(offsets) - 1, trailing)
        for b in range(len(offsets) - 1):
            rows = flat[offsets[b]:offsets[b + 1]]
            if rows.shape[0] == 0:
                assert np.all(got[b] == np.iinfo(np.uint64).max)
            else:
                winner = rows.argmin(axis=0) if name == "ArgMin" else rows.argmax(axis=0)  # first occurrence = lowest index
                np.testing.assert_array_equal(got[b], (offsets[b] + winner) * trailing + np.arange(trailing), err_msg=f"{name} segment {b}")


def awkward_offsets(rows):
    """Partitions that put every case of the segment kernels side by side: empty segments at position 0, at multiples of the
    lane ranges and chunks (16, 64, 256 rows), runs of one-row segments, a segment that spans many chunks, rows after the
    last segment."""
    cuts = [0, 0, 0, 1, 2, 3, 3, 16, 16, 40, 64, 64, 64, 100, 256, 256, 300, 301, 302, 303, 512, 1800, 1800, 2047, 2048, 2048, 2600]
    cuts = [c for c in cuts if c <= rows]
    return np.array(cuts + [min(rows, 2900)] * 3, dtype=np.int64)


AWKWARD_SHAPES = [((3000, 64), DataType.fp32), ((3000, 200), DataType.fp16), ((2100, 3), DataType.fp32), ((3000, 512), DataType.bf16)]
# both kernels over every shape; the other block sizes and walking groups of the by-rows kernel over one shape each
SEGMENT_KERNELS = [(k, {}, s, d) for k in ("teams", "rows") for s, d in AWKWARD_SHAPES] + [
    ("rows", {"THOR_SEGMENT_THREADS": "64"}, *AWKWARD_SHAPES[0]), ("rows", {"THOR_SEGMENT_GROUP": "16", "THOR_SEGMENT_BATCH": "8"}, *AWKWARD_SHAPES[1]),
    ("rows", {"THOR_SEGMENT_GROUP": "2", "THOR_SEGMENT_THREADS": "128"}, *AWKWARD_SHAPES[3])]


@pytest.mark.parametrize("kernel,switches,shape,dtype", SEGMENT_KERNELS,
                         ids=[f"{k}" + "".join(f"-{n[13:].lower()}{v}" for n, v in e.items()) + f"-{s[0]}x{s[1]}-{d.name}" for k, e, s, d in SEGMENT_KERNELS])
def test_both_segment_kernels_on_awkward_partitions(stream, monkeypatch, kernel, switches, shape, dtype):
    """The planner picks between two kernels (segments dealt out to teams of lanes, rows dealt out to lanes) by the shape; the
    tuning switches force each of them, and other block sizes and walking groups, on the same partitions."""
    monkeypatch.setenv("THOR_SEGMENT_KERNEL", kernel)
    for name, value in switches.items():
        monkeypatch.setenv(name, value)
    rng = np.random.default_rng(shape[1])
    x = to_storage(rng.standard_normal(shape).astype(np.float32), dtype)
    x[5, 0] = x[1900, 1] = to_storage(np.array([np.nan], np.float32), dtype)[0]
    xf = from_storage(x, dtype).astype(np.float64)
    offsets = awkward_offsets(shape[0])
    tx = copy_numpy_to_gpu(x, stream, dtype)
    for offsets_dtype in (DataType.uint32, DataType.uint64):
        toff = upload_offsets(offsets, stream, offsets_dtype)
        lengths = np.diff(offsets).reshape(-1, 1)
        wide = offsets_dtype == DataType.uint64  # 64-bit offsets change how the partition is read, not what is folded: two operations
        for name, op in VALUE_OPS.items():
            if wide and name != "Mean":
                continue
            stamped = ph.CubSegmentedReduction(op, DataType.fp32).stamp(tx, toff, stream)
            assert ("by_rows" if kernel == "rows" else "by_teams") in stamped.get_kernel_variant()
            stamped.run()
            got = gpu_to_f32(stamped.get_output_tensor(), stream).astype(np.float64)
            want = segment_reference(xf, offsets, name)
            if name in ("Min", "Max"):
                np.testing.assert_array_equal(got, want, err_msg=f"{name} {stamped.get_kernel_variant()}")
            else:
                absolute = segment_reference(np.abs(np.nan_to_num(xf)), offsets, "Sum") / (np.maximum(lengths, 1) if name == "Mean" else 1)
                assert np.array_equal(np.isnan(got), np.isnan(want)), f"{name} {stamped.get_kernel_variant()}"
                assert np.all(np.isnan(want) | (np.abs(got - want) <= 1e-5 * absolute + 1e-30)), f"{name} {stamped.get_kernel_variant()}"
        for name, op in ARG_OPS.items():
            if wide and name != "ArgMax":
                continue
            stamped = ph.CubSegmentedArgReduction(op).stamp(tx, toff, stream)
            stamped.run()
            got = copy_gpu_to_numpy(stamped.get_index_output_tensor(), stream).reshape(len(offsets) - 1, shape[1])
            for b in range(len(offsets) - 1):
                rows = xf[offsets[b]:offsets[b + 1]]
                if rows.shape[0] == 0:
                    assert np.all(got[b] == np.iinfo(np.uint64).max), f"{name} empty segment {b}"
                else:
                    winner = rows.argmin(axis=0) if name == "ArgMin" else rows.argmax(axis=0)  # numpy: the first NaN wins, else the first best
                    np.testing.assert_array_equal(got[b], (offsets[b] + winner) * shape[1] + np.arange(shape[1]), err_msg=f"{name} segment {b} {stamped.get_kernel_variant()}")


@pytest.mark.parametrize("seed", range(6))
def test_random_partitions_give_the_same_answer_through_both_kernels(stream, monkeypatch, seed):
    """Random partitions with many empty and one-row segments, rows of 1 to 260 elements: maxima and winners must agree bit for
    bit between the two segment kernels and with numpy, sums within the accumulation-order tolerance."""
    rng = np.random.default_rng(1000 + seed)
    rows = int(rng.integers(1, 6000))
    width = int(rng.choice([1, 2, 3, 16, 48, 64, 130, 260]))
    segments = int(rng.integers(1, 400))
    style = seed % 3
    if style == 0:
        cuts = np.sort(rng.integers(0, rows + 1, segments - 1)) if segments > 1 else np.array([], np.int64)
    elif style == 1:  # geometric lengths: mostly tiny segments, a few long ones
        lengths = rng.geometric(0.3, segments) - 1
        cuts = np.minimum(np.cumsum(lengths)[:-1], rows) if segments > 1 else np.array([], np.int64)
    else:  # one long segment among empties
        cuts = np.sort(rng.choice([0, rows // 3, rows], segments - 1)) if segments > 1 else np.array([], np.int64)
    last = int(rng.integers(cuts[-1] if len(cuts) else 0, rows + 1))
    offsets = np.concatenate([[0], cuts, [last]]).astype(np.int64)
    dtype = [DataType.fp32, DataType.fp16, DataType.bf16][seed % 3]
    x = to_storage(rng.integers(-6, 7, (rows, width)).astype(np.float32) / 4, dtype)  # few distinct values: ties everywhere
    xf = from_storage(x, dtype).astype(np.float64)
    tx = copy_numpy_to_gpu(x, stream, dtype)
    toff = upload_offsets(offsets, stream)
    results = {}
    for kernel in ("teams", "rows"):
        monkeypatch.setenv("THOR_SEGMENT_KERNEL", kernel)
        stamped = ph.CubSegmentedReduction(ph.CubReductionOp.Max, DataType.fp32).stamp(tx, toff, stream)
        stamped.run()
        maxima = gpu_to_f32(stamped.get_output_tensor(), stream)
        stamped = ph.CubSegmentedReduction(ph.CubReductionOp.Sum, DataType.fp32).stamp(tx, toff, stream)
        stamped.run()
        sums = gpu_to_f32(stamped.get_output_tensor(), stream)
        stamped = ph.CubSegmentedArgReduction(ph.CubArgReductionOp.ArgMin, DataType.uint32).stamp(tx, toff, stream)
        stamped.run()
        winners = copy_gpu_to_numpy(stamped.get_index_output_tensor(), stream)
        results[kernel] = (maxima, sums, winners)
    np.testing.assert_array_equal(results["teams"][0], results["rows"][0])
    np.testing.assert_array_equal(results["teams"][2], results["rows"][2])
    np.testing.assert_array_equal(results["rows"][0].reshape(segments, width), segment_reference(xf, offsets, "Max").astype(np.float32))
    np.testing.assert_array_equal(results["rows"][1].reshape(segments, width), segment_reference(xf, offsets, "Sum").astype(np.float32))  # quarters: exact
    flat = xf.reshape(rows, width)
    got = results["rows"][2].reshape(segments, width)
    for b in range(segments):
        piece = flat[offsets[b]:offsets[b + 1]]
        if piece.shape[0] == 0:
            assert np.all(got[b] == np.iinfo(np.uint32).max)
        else:
            np.testing.assert_array_equal(got[b], (offsets[b] + piece.argmin(axis=0)) * width + np.arange(width))


def test_offsets_are_read_at_run_time_and_outputs_are_reused(stream):
    """CubOffsetSegmentedReductionTest.cpp:239-295: runtime offsets are not inspected by the stamp; a stamped reduction follows the
    partition that is in the offsets tensor when it runs."""
    x = copy_numpy_to_gpu(np.array([1, 2, 3, 4, 5, 6], np.float32), stream, DataType.fp32)
    offsets = upload_offsets([7, 7, 7, 7], stream)  # not a valid partition yet
    out = gpu_tensor([3], DataType.fp32)
    with pytest.raises(ValueError):
        ph.CubSegmentedReduction(ph.CubReductionOp.Mean, DataType.fp32).stamp(x, offsets, stream, preallocated_output=out)
    stamped = ph.CubSegmentedReduction(ph.CubReductionOp.Mean, DataType.fp32).stamp_runtime_offsets(x, out, offsets, stream)
    for partition, want in (([0, 2, 2, 6], [1.5, 0.0, 4.5]), ([0, 1, 4, 6], [1.0, 3.0, 5.5])):
        host = ph.PhysicalTensor(ph.Placement(ph.DeviceType.cpu), ph.PhysicalTensor.Descriptor(DataType.uint32, [4]))
        host.numpy()[...] = np.array(partition, np.uint32)
        offsets.copy_from_async(host, stream)
        stamped.run()
        np.testing.assert_array_equal(copy_gpu_to_numpy(out, stream), np.array(want, np.float32))
    assert stamped.get_output_tensor().mem_ptr() == out.mem_ptr()


def test_nan_propagates_per_component_and_output_dtypes(stream):
    x = np.array([[1.0, np.nan], [2.0, 5.0], [3.0, 4.0], [np.nan, 1.0]], dtype=np.float32)
    tx = copy_numpy_to_gpu(x, stream, DataType.fp32)
    offsets = upload_offsets([0, 2, 4], stream)
    for op, pick in ((ph.CubReductionOp.Min, np.minimum), (ph.CubReductionOp.Max, np.maximum)):
        stamped = ph.CubSegmentedReduction(op, DataType.fp32).stamp(tx, offsets, stream)
        stamped.run()
        got = gpu_to_f32(stamped.get_output_tensor(), stream)
        assert np.isnan(got[0, 1]) and np.isnan(got[1, 0]) and got[0, 0] == pick(1.0, 2.0) and got[1, 1] == pick(4.0, 1.0)
    big = copy_numpy_to_gpu(np.full((4,), 300.0, np.float32), stream, DataType.fp32)
    for od, want in ((DataType.fp16, 600.0), (DataType.bf16, 600.0), (DataType.fp8_e4m3, 448.0)):
        stamped = ph.CubSegmentedReduction(ph.CubReductionOp.Sum, od).stamp(big, offsets, stream)
        stamped.run()
        assert stamped.get_output_tensor().get_data_type() == od
        np.testing.assert_array_equal(gpu_to_f32(stamped.get_output_tensor(), stream), np.array([want, want], np.float32))


def test_contract_violations_raise_value_errors(stream):
    """CubOffsetSegmentedReductionTest.cpp:457-511."""
    x = copy_numpy_to_gpu(np.array([1, 2, 3, 4], np.float32), stream, DataType.fp32)
    x2 = copy_numpy_to_gpu(np.array([[1, 2], [3, 4]], np.float32), stream, DataType.fp32)
    good = upload_offsets([0, 2, 4], stream)
    with pytest.raises(ValueError, match="sum, mean, min, and max"):
        ph.CubSegmentedReduction(ph.CubReductionOp.Product).stamp(x, good, stream)
    for bad in ([0, 1, 3],):
        with pytest.raises(ValueError):
            ph.CubSegmentedReduction(ph.CubReductionOp.Sum).stamp(x2, upload_offsets(bad, stream), stream)
    with pytest.raises(ValueError, match="UINT32 or UINT64"):
        ph.CubSegmentedReduction(ph.CubReductionOp.Sum).stamp(x, copy_numpy_to_gpu(np.array([0, 2, 4], np.float32), stream, DataType.fp32), stream)
    for bad, message in (([0], "rank 1"), ([1, 2, 4], "start at 0"), ([0, 3, 2], "non-decreasing"), ([0, 2, 5], "exceed")):
        with pytest.raises(ValueError, match=message):
            ph.CubSegmentedReduction(ph.CubReductionOp.Sum).stamp(x, upload_offsets(bad, stream), stream)
    with pytest.raises(ValueError, match="shape"):
        ph.CubSegmentedReduction(ph.CubReductionOp.Sum, DataType.fp32).stamp(x2, upload_offsets([0, 1, 2], stream), stream,
                                                                             preallocated_output=gpu_tensor([2, 1, 2], DataType.fp32))
    with pytest.raises(ValueError, match="shape"):
        ph.CubSegmentedReduction(ph.CubReductionOp.Sum, DataType.fp32).stamp(x, good, stream, preallocated_output=gpu_tensor([2, 2], DataType.fp32))
    with pytest.raises(ValueError, match="shape"):
        ph.CubSegmentedArgReduction(ph.CubArgReductionOp.ArgMin, DataType.uint32).stamp(x2, upload_offsets([0, 1, 2], stream), stream,
                                                                                        preallocated_index_output=gpu_tensor([2], DataType.uint32))


@pytest.mark.parametrize("shape", [(3 * 4096 + 17,), (1500, 40), (9000, 3)], ids=str)
def test_segments_that_begin_and_end_on_block_boundaries(stream, shape):
    """The kernel streams fixed chunks of rows (chunk_rows in the variant text) and stitches segments that span chunks:
    segments that begin or end exactly on a chunk boundary, empty segments on boundaries and at both ends, one segment
    covering several whole chunks, and rows after the last segment that belong to nobody."""
    import re
    rng = np.random.default_rng(7)
    x = rng.standard_normal(shape).astype(np.float32)
    tx = copy_numpy_to_gpu(x, stream, DataType.fp32)
    probe = ph.CubSegmentedReduction(ph.CubReductionOp.Sum, DataType.fp32).stamp(tx, upload_offsets([0, shape[0]], stream), stream)
    chunk = int(re.search(r"chunk_rows=(\d+)", probe.get_kernel_variant()).group(1))
    assert shape[0] > 2 * chunk, probe.get_kernel_variant()
    n = shape[0]
    partitions = [
        [0, 0, chunk, chunk, chunk, 2 * chunk, 2 * chunk + 1, n, n, n],
        [0, chunk - 1, chunk + 1, 2 * chunk, n - 3],
        [0, 0, 0, n],
        [0, 1, 2 * chunk, 2 * chunk, n - 1, n],
        [0, chunk, 2 * chunk, n],
        [0, 0],
    ]
    trailing = int(np.prod(shape[1:])) if len(shape) > 1 else 1
    for partition in partitions:
        # empty segments after the last one bring every partition to ten offsets: the kernels bake the segment count in, so the
        # partitions share their compiled kernels
        partition = partition + [partition[-1]] * (10 - len(partition))
        offsets = np.array(partition, dtype=np.int64)
        toff = upload_offsets(offsets, stream, DataType.uint64)
        for name, op in VALUE_OPS.items():
            if name == "Min":
                continue
            stamped = ph.CubSegmentedReduction(op, DataType.fp32).stamp(tx, toff, stream)
            stamped.run()
            got = gpu_to_f32(stamped.get_output_tensor(), stream).astype(np.float64)
            want = segment_reference(x.astype(np.float64), offsets, name)
            if name in ("Min", "Max"):
                np.testing.assert_array_equal(got, want, err_msg=f"{name} {partition}")
            else:
                scale = segment_reference(np.abs(x).astype(np.float64), offsets, "Sum")
                if name == "Mean":
                    scale = scale / np.maximum(np.diff(offsets), 1).reshape([-1] + [1] * (len(shape) - 1))
                assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-30), f"{name} {partition}"
        flat = x.reshape(n, trailing)
        for name, op in ARG_OPS.items():
            if name == "ArgMax":
                continue
            stamped = ph.CubSegmentedArgReduction(op, DataType.uint32).stamp(tx, toff, stream)
            stamped.run()
            got = copy_gpu_to_numpy(stamped.get_index_output_tensor(), stream).reshape(len(offsets) - 1, trailing)
            for b in range(len(offsets) - 1):
                rows = flat[offsets[b]:offsets[b + 1]]
                if rows.shape[0] == 0:
                    assert np.all(got[b] == np.iinfo(np.uint32).max), f"{name} {partition} segment {b}"
                else:
                    winner = rows.argmin(axis=0) if name == "ArgMin" else rows.argmax(axis=0)
                    np.testing.assert_array_equal(got[b], (offsets[b] + winner) * trailing + np.arange(trailing), err_msg=f"{name} {partition} segment {b}")
