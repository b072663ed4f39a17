"""Random differential runs of the GPU kernels against the oracle, outside the collected suite (every case compiles its own kernels,
0.3-1 s each on a cold box):

    python tests/soak_against_oracle.py FAMILY SEED CASES      FAMILY: backward | ragged | rope | views | expressions | conversions | topk | topk_rows | scans | reductions | rows

Shapes, dtypes, operations, orders and data kinds (normal, few levels, sorted either way, a narrow band, outliers over zeros, NaN /
inf / signed zeros, a repeated block) are drawn at random; every case is printed before it runs and checked with the same helper
the collected test of its family uses (bit-exact for selections, scans of exact operations, min / max and arg reductions; the
tests' tolerances for float sums).  The first failure ends the run with the case on the last line.  This is the run that showed
the 64-bit shift defect of the device (row top-k, sorted fp16 rows: tests/test_selection_gpu.py keeps that case)."""
from __future__ import annotations

import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

from helpers import to_storage  # noqa: E402
from thor_amd import physical as ph  # noqa: E402
from thor_amd.dtypes import DataType, numpy_carrier  # noqa: E402
from thor_amd.physical import ScanOp  # noqa: E402

FLOATS = (DataType.fp16, DataType.bf16, DataType.fp32)
KINDS = ["normal", "levels", "sorted", "reversed", "narrow", "outliers", "specials", "blocks"]


def keys_of(rng, dtype, rows, size, kind, k):
    """[rows, size] keys of one data kind (sorted kinds are sorted inside every row)."""
    n = rows * size
    if dtype in FLOATS:
        if kind == "normal":
            v = rng.standard_normal(n).astype(np.float32) * 100
        elif kind == "levels":
            v = np.round(rng.standard_normal(n) * rng.integers(1, 40)).astype(np.float32)
        elif kind in ("sorted", "reversed"):
            v = np.sort(rng.standard_normal((rows, size)).astype(np.float32), axis=1)
            v = (v[:, ::-1] if kind == "reversed" else v).reshape(-1).copy()
        elif kind == "narrow":
            v = (1.0 + rng.random(n) * 2.0 ** -rng.integers(4, 20)).astype(np.float32) * (1 if rng.random() < 0.5 else -1)
        elif kind == "outliers":
            v = np.zeros(n, np.float32)
            at = rng.integers(0, n, max(k // 2, 1))
            v[at] = rng.standard_normal(at.size).astype(np.float32) * 50
        elif kind == "specials":
            v = rng.standard_normal(n).astype(np.float32)
            at = rng.integers(0, n, max(n // 50, 1))
            v[at] = rng.choice(np.array([np.inf, -np.inf, np.nan, 0.0, -0.0], np.float32), at.size)
        else:
            block = rng.standard_normal(min(1 << 16, n)).astype(np.float32)
            v = np.tile(block, n // block.size + 1)[:n].copy()
        return to_storage(v, dtype)
    carrier = numpy_carrier(dtype)
    info = np.iinfo(carrier)
    if kind in ("levels", "narrow"):
        return rng.integers(0, int(rng.integers(2, 50)), n).astype(carrier)
    if kind in ("sorted", "reversed"):
        v = np.sort(rng.integers(info.min, int(info.max) + 1, (rows, size)).astype(carrier), axis=1)
        return (v[:, ::-1] if kind == "reversed" else v).reshape(-1).copy()
    if kind == "outliers":
        v = np.zeros(n, carrier)
        at = rng.integers(0, n, max(k // 2, 1))
        v[at] = rng.integers(info.min, int(info.max) + 1, at.size)
        return v
    return rng.integers(info.min, int(info.max) + 1, n).astype(carrier)


def topk_case(rng, stream):
    import test_selection_gpu as T
    dtype = [DataType.fp32, DataType.fp32, DataType.bf16, DataType.fp16, DataType.int32, DataType.uint32, DataType.uint16, DataType.int16][rng.integers(0, 8)]
    n = int(rng.integers(1 << 20, 1 << 23)) if rng.random() < 0.8 else int(rng.integers(1 << 23, 1 << 25))
    if rng.random() < 0.5:
        n = n // 4 * 4
    k = int(max(1, 2 ** rng.uniform(0, np.log2(max(n // 256, 1)))))
    largest, pairs, kind = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), KINDS[rng.integers(0, len(KINDS))]
    print(f"{dtype.name} n={n} k={k} largest={largest} pairs={pairs} kind={kind}", flush=True)
    keys = keys_of(rng, dtype, 1, n, kind, k)
    got, got_values, variant = T.run_top_k(keys, dtype, k, largest, stream, pairs=pairs)
    T.check_top_k(keys, dtype, k, largest, got, got_values)
    return variant


def topk_rows_case(rng, stream):
    import test_selection_gpu as T
    dtype = [DataType.fp32, DataType.bf16, DataType.fp16, DataType.int32, DataType.uint16, DataType.int8, DataType.uint8][rng.integers(0, 7)]
    size = min(int(2 ** rng.uniform(1, 13.2)), 8192)
    if rng.random() < 0.4:
        size = max(size // 8 * 8, 8)
    rows = int(max(1, min(2 ** rng.uniform(0, 14), (1 << 22) // size)))
    k = int(max(1, min(size - 1, 2 ** rng.uniform(0, np.log2(size)))))
    largest, pairs, kind = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), KINDS[rng.integers(0, 5)]
    print(f"{dtype.name} rows={rows} size={size} k={k} largest={largest} pairs={pairs} kind={kind}", flush=True)
    keys = keys_of(rng, dtype, rows, size, kind, k)
    got, got_values, variant = T.run_top_k(keys, dtype, k, largest, stream, pairs=pairs, segment_size=size)
    T.check_top_k(keys, dtype, k, largest, got, got_values, segment_size=size)
    return variant


def scans_case(rng, stream):
    import oracle
    import test_scan_gpu as S
    import test_selection_gpu as T
    what = ["rows", "flat", "segments", "select"][rng.integers(0, 4)]
    if what == "select":
        dtype = [DataType.fp32, DataType.fp16, DataType.uint8, DataType.int32, DataType.uint16][rng.integers(0, 5)]
        n = int(2 ** rng.uniform(0, 23))
        density = [0.0, 1.0, 0.5, 0.01, 0.99, rng.random()][rng.integers(0, 6)]
        flag_dtype = [DataType.uint8, DataType.boolean][rng.integers(0, 2)]
        print(f"select {dtype.name} n={n} density={density:.3f} flags={flag_dtype.name}", flush=True)
        values = T.random_keys(rng, n, dtype)
        flags = (rng.random(n) < density).astype(np.uint8) * (rng.integers(1, 255, n).astype(np.uint8) if flag_dtype == DataType.uint8 else 1)
        out, count, variant = T.run_select(values, flags, dtype, flag_dtype, stream)
        want = values[flags != 0]
        assert count == want.size, (count, want.size)
        np.testing.assert_array_equal(T.bits_of(out[:count]), T.bits_of(want))
        return variant
    dtype = [DataType.uint32, DataType.fp32, DataType.fp16, DataType.bf16][rng.integers(0, 4)]
    op = [ScanOp.sum, ScanOp.min, ScanOp.max, ScanOp.product, ScanOp.arg_min, ScanOp.arg_max][rng.integers(0, 6)]
    if what == "segments" and op == ScanOp.product:
        op = ScanOp.sum
    inclusive, reverse = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    if what == "rows":
        cols = int(2 ** rng.uniform(0, 17))
        shape = (int(max(1, min(2 ** rng.uniform(0, 12), (1 << 22) // cols))), cols)
    else:
        shape = (1, int(2 ** rng.uniform(0, 23.5))) if what == "flat" else (int(2 ** rng.uniform(4, 22)),)
    n = int(np.prod(shape))
    if dtype == DataType.uint32:
        carrier = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32) if op != ScanOp.product else rng.integers(1, 4, n).astype(np.uint32)
    elif op == ScanOp.product:  # signed powers of two whose running exponent stays small: exact in any order
        steps = np.diff(np.concatenate([[0], np.clip(np.cumsum(rng.integers(-1, 2, n)), -6, 6)]))
        carrier = to_storage((np.exp2(steps) * rng.choice([1.0, -1.0], n)).astype(np.float32), dtype)
    else:
        carrier = to_storage((np.round(rng.standard_normal(n) * 8) / 8).astype(np.float32), dtype)
    carrier = carrier.reshape(shape)
    if what == "segments":
        segments = int(max(1, min(2 ** rng.uniform(0, 16), n)))
        cuts = np.sort(rng.integers(0, n + 1, segments))
        offsets = np.concatenate([[0], cuts, [max(n - int(rng.integers(0, 50)), int(cuts[-1]))]])
        width = [DataType.uint32, DataType.uint64][rng.integers(0, 2)]
        print(f"segments {dtype.name} n={n} segments={segments} {op.name} inclusive={inclusive} reverse={reverse} offsets={width.name}", flush=True)
        got, variant = S.run_scan(carrier, dtype, stream, op, inclusive, reverse, offsets=offsets, offsets_dtype=width)
        active = int(offsets[-1])
        if dtype == DataType.uint32 or op != ScanOp.sum:
            expected = oracle.scan(carrier, S.ORACLE_OP[op], inclusive, reverse, offsets=offsets, dtype=int(dtype))
            np.testing.assert_array_equal(got[:active], expected[:active])
        else:
            S.check(got[:active], carrier[:active], dtype, op, inclusive, reverse, offsets=offsets)
        return variant
    segment_size = shape[1] if what == "rows" else 0
    print(f"{what} {dtype.name} shape={shape} {op.name} inclusive={inclusive} reverse={reverse}", flush=True)
    got, variant = S.run_scan(carrier, dtype, stream, op, inclusive, reverse, segment_size=segment_size)
    S.check(got, carrier, dtype, op, inclusive, reverse, segment_size=segment_size)
    return variant


def reductions_case(rng, stream):
    import test_reduction_gpu as R
    import test_segmented_reduction_gpu as SR
    what = ["value", "arg", "segments"][rng.integers(0, 3)]
    if what == "segments":
        rank = int(rng.integers(1, 4))
        rest = [int(2 ** rng.uniform(0, 6)) for _ in range(rank - 1)]
        rows = int(2 ** rng.uniform(3, 17))
        while rows * int(np.prod(rest or [1])) > (1 << 21):
            rows //= 2
        shape = tuple([max(rows, 8)] + rest)
        segments = int(max(6, min(2 ** rng.uniform(2, 12), shape[0])))
        dtype = [DataType.fp32, DataType.bf16, DataType.fp16, DataType.fp8_e4m3][rng.integers(0, 4)]
        print(f"segments shape={shape} segments={segments} {dtype.name}", flush=True)
        SR.test_random_ragged_partitions_against_numpy(stream, shape, segments, dtype)
        return ""
    rank = int(rng.integers(1, 5))
    left = 2 ** rng.uniform(0, 22)
    dims = []
    for d in range(rank):
        extent = int(max(1, round(left if d == rank - 1 else 2 ** rng.uniform(0, np.log2(max(left, 1.0001))))))
        if rng.random() < 0.3:
            extent |= 1
        dims.append(extent)
        left = max(left / extent, 1)
    axes = sorted(rng.choice(rank, int(rng.integers(1, rank + 1)), replace=False).tolist())
    dtype = [DataType.fp32, DataType.fp16, DataType.bf16][rng.integers(0, 3)]
    print(f"{what} dims={dims} axes={axes} {dtype.name}", flush=True)
    if what == "value":
        R.test_value_ops_against_oracle(stream, dims, axes, dtype)
    else:
        R.test_arg_ops_against_oracle_with_ties_and_nans(stream, dims, axes)
    return ""


def rows_case(rng, stream):
    import test_row_fusion_gpu as RF
    cols = int(2 ** rng.uniform(1, 15))
    rows = int(max(2, min(2 ** rng.uniform(1, 13), (1 << 22) // cols)))
    dtype = [DataType.fp32, DataType.fp16, DataType.bf16][rng.integers(0, 3)]
    if rng.random() < 0.5:
        print(f"softmax {(rows, cols)} {dtype.name}", flush=True)
        RF.test_softmax_single_pass_matches_staged_and_closed_form(None, dtype, (rows, cols))
    else:
        cols = min(cols, 8192)
        shape = (rows, cols) if rng.random() < 0.6 else (max(rows // 3, 1), 3, cols)
        print(f"normalise {shape} {dtype.name}", flush=True)
        RF.test_mean_variance_normalisation_single_pass(None, dtype, shape)
    return ""


def conversions_case(rng, stream):
    """Out of place and in place, random lengths and element offsets at both ends, guard bytes around the destination."""
    import oracle
    import test_convert_gpu as C
    from thor_amd.dtypes import size_of
    from thor_amd.runtime import DeviceBuffer, TypeConverter
    src, dst = [C.ALL[i] for i in rng.choice(len(C.ALL), 2, replace=False)]
    n = int(2 ** rng.uniform(0, 21))
    in_place = rng.random() < 0.3
    src_off, dst_off = (0, 0) if in_place else (int(rng.integers(0, 9)), int(rng.integers(0, 9)))
    wide = src in (DataType.int64, DataType.uint64, DataType.int32, DataType.uint32) and dst in C.FLOATS and rng.random() < 0.5
    print(f"{src.name} -> {dst.name} n={n} in_place={in_place} offsets={src_off},{dst_off} wide={wide}", flush=True)
    x = np.resize(C.wide_integers(src, rng), n) if wide else C._sample_for(src, dst, n, rng)
    want = oracle.convert(x, int(src), int(dst))
    ssz, dsz = size_of(src), size_of(dst)
    if in_place:
        buf = DeviceBuffer(n * max(ssz, dsz) + 256)
        guard = np.full(256, 0xA5, np.uint8)
        buf.upload(guard, offset_bytes=n * max(ssz, dsz))
        buf.upload(x)
        TypeConverter.convert_type(buf.ptr, buf.ptr, src, dst, n)
        got = buf.download(numpy_carrier(dst), n)
        assert np.array_equal(buf.download(np.uint8, 256, offset_bytes=n * max(ssz, dsz)), guard), "wrote past the end"
    else:
        a, b = DeviceBuffer((n + src_off) * ssz + 256), DeviceBuffer((n + dst_off) * dsz + 512)
        fill = np.full((n + dst_off) * dsz + 512, 0x5A, np.uint8)
        b.upload(fill)
        a.upload(x, offset_bytes=src_off * ssz)
        TypeConverter.convert_type(a.ptr + src_off * ssz, b.ptr + 256 + dst_off * dsz, src, dst, n)
        got = b.download(numpy_carrier(dst), n, offset_bytes=256 + dst_off * dsz)
        assert np.all(b.download(np.uint8, 256 + dst_off * dsz) == 0x5A), "wrote before the destination"
        assert np.all(b.download(np.uint8, 256 - dst_off * dsz, offset_bytes=256 + (dst_off + n) * dsz) == 0x5A), "wrote past the destination"
    C.assert_same_bits(got, want, dst)
    return ""


def expressions_case(rng, stream):
    """Fused elementwise expressions over broadcast operands, with or without a reduction over some axes at the end.  Operands hold
    small integers and the tree keeps every intermediate below 200 in magnitude, so fp32, fp16 and bf16 arithmetic is exact in any
    order and the result must equal NumPy's integer arithmetic bit for bit."""
    from helpers import from_storage, run_staged
    ex = ph.Expression
    rank = int(rng.integers(1, 5))
    left = 2 ** rng.uniform(0, 20)
    dims = []
    for d in range(rank):
        extent = int(max(1, round(left if d == rank - 1 else 2 ** rng.uniform(0, np.log2(max(left, 1.0001))))))
        dims.append(extent)
        left = max(left / extent, 1)
    dtype = [DataType.fp32, DataType.fp16, DataType.bf16][rng.integers(0, 3)]
    names = "abcd"[:int(rng.integers(2, 5))]
    arrays, nodes = {}, []
    for i, name in enumerate(names):
        shape = [e if i == 0 or rng.random() < 0.7 else 1 for e in dims]
        values = rng.integers(-3, 4, shape)
        arrays[name] = to_storage(values.astype(np.float32), dtype)
        nodes.append((ex.input(name), values.astype(np.int64), 3))
    text = list(names)
    used = [{name} for name in names]
    for _ in range(int(rng.integers(1, 6))):
        i, j = int(rng.integers(0, len(nodes))), int(rng.integers(0, len(nodes)))
        (x, xv, xb), (y, yv, yb) = nodes[i], nodes[j]
        op = ["add", "sub", "mul", "min", "max", "where", "neg", "abs"][rng.integers(0, 8)]
        if op == "mul" and xb * yb > 200 or op in ("add", "sub") and xb + yb > 200:
            op = "max"
        if op == "add":
            node = (x + y, xv + yv, xb + yb)
        elif op == "sub":
            node = (x - y, xv - yv, xb + yb)
        elif op == "mul":
            node = (x * y, xv * yv, xb * yb)
        elif op == "min":
            node = (x.min(y), np.minimum(xv, yv), max(xb, yb))
        elif op == "max":
            node = (x.max(y), np.maximum(xv, yv), max(xb, yb))
        elif op == "where":
            node = (ex.where(x > y, x, y - 1.0), np.where(xv > yv, xv, yv - 1), max(xb, yb) + 1)
        elif op == "neg":
            node = (-x, -xv, xb)
        else:
            node = (x.abs(), np.abs(xv), xb)
        nodes.append(node)
        text.append(f"{op}({text[i]},{text[j]})" if op not in ("neg", "abs") else f"{op}({text[i]})")
        used.append(used[i] | used[j] if op not in ("neg", "abs") else set(used[i]))
    expr, want, bound = nodes[-1]
    for name in names:  # every input takes part, so that the plan binds all of them
        if name not in used[-1]:
            k = names.index(name)
            expr, want, bound = expr.max(nodes[k][0]), np.maximum(want, nodes[k][1]), max(bound, 3)
            text[-1] = f"max({text[-1]},{name})"
    want = np.broadcast_to(want, np.broadcast_shapes(*[arrays[n].shape for n in names])).copy()
    reduce = None
    if rng.random() < 0.5:
        axes = sorted(rng.choice(rank, int(rng.integers(1, rank + 1)), replace=False).tolist())
        count = int(np.prod([want.shape[a] for a in axes]))
        reduce = ["sum", "max", "min"][rng.integers(0, 3)]
        if reduce == "sum" and count * bound >= (1 << 24):
            reduce = "max"
        expr = {"sum": expr.reduce_sum, "max": expr.reduce_max, "min": expr.reduce_min}[reduce](axes)
        want = {"sum": np.sum, "max": np.max, "min": np.min}[reduce](want, axis=tuple(axes), keepdims=True)
        text[-1] = f"{reduce}{axes}({text[-1]})"
    print(f"{dtype.name} dims={dims} shapes={[list(arrays[n].shape) for n in names]} {text[-1]}", flush=True)
    plan, outs = run_staged(expr, arrays, dtype)
    got = outs["output"]
    got = got.astype(np.float64) if reduce else from_storage(got, dtype).astype(np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    np.testing.assert_array_equal(got, want.astype(np.float64), err_msg=str(plan.stage_descriptions()))
    return " | ".join(plan.stage_kind_names())


def views_case(rng, stream):
    """An operand seen through a permuted (and possibly cropped) strided view, in elementwise work with a dense operand and under a
    reduction over random axes; small integers, so that the result equals NumPy's bit for bit."""
    from helpers import from_storage, run_staged
    ex = ph.Expression
    rank = int(rng.integers(2, 5))
    left = 2 ** rng.uniform(2, 19)
    dims = []
    for d in range(rank):
        extent = int(max(1, round(left if d == rank - 1 else 2 ** rng.uniform(0, np.log2(max(left, 1.0001))))))
        dims.append(extent)
        left = max(left / extent, 1)
    dtype = [DataType.fp32, DataType.fp16, DataType.bf16][rng.integers(0, 3)]
    x = rng.integers(-3, 4, dims)
    strides = [int(np.prod(dims[d + 1:])) for d in range(rank)]
    perm = rng.permutation(rank).tolist()
    crop = [int(rng.integers(0, dims[a])) if rng.random() < 0.3 and dims[a] > 1 else 0 for a in range(rank)]  # first index kept, per storage axis
    view_dims = [dims[a] - crop[a] for a in perm]
    view_strides = [strides[a] for a in perm]
    offset = sum(crop[a] * strides[a] for a in range(rank))
    seen = x[tuple(slice(crop[a], None) for a in range(rank))].transpose(perm)
    y = rng.integers(-3, 4, view_dims)
    view = ex.input("x").strided_view(view_dims, view_strides, offset)
    expr, want = view * ex.input("y") + view, seen * y + seen
    text = f"x{dims} perm={perm} crop={crop}"
    reduced = rng.random() < 0.6
    if reduced:
        axes = sorted(rng.choice(rank, int(rng.integers(1, rank + 1)), replace=False).tolist())
        op = ["sum", "max", "min"][rng.integers(0, 3)]
        if op == "sum" and int(np.prod([view_dims[a] for a in axes])) * 12 >= (1 << 24):
            op = "max"
        expr = {"sum": expr.reduce_sum, "max": expr.reduce_max, "min": expr.reduce_min}[op](axes)
        want = {"sum": np.sum, "max": np.max, "min": np.min}[op](want, axis=tuple(axes), keepdims=True)
        text += f" {op}{axes}"
    print(f"{dtype.name} {text}", flush=True)
    plan, outs = run_staged(expr, {"x": to_storage(x.astype(np.float32), dtype), "y": to_storage(y.astype(np.float32), dtype)}, dtype)
    got = outs["output"]
    got = got.astype(np.float64) if reduced else from_storage(got, dtype).astype(np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    np.testing.assert_array_equal(got, want.astype(np.float64), err_msg=str(plan.stage_descriptions()))
    return " | ".join(plan.stage_kind_names())


def ragged_case(rng, stream):
    """Ragged softmax / centering through the expression planner and the segmented broadcast, on random partitions."""
    import test_ragged_expression_gpu as RE
    import test_segmented_broadcast_gpu as SB
    rank = int(rng.integers(1, 4))
    rest = tuple(int(2 ** rng.uniform(0, 5)) for _ in range(rank - 1))
    rows = int(2 ** rng.uniform(5, 17))
    while rows * int(np.prod(rest or (1,))) > (1 << 20):
        rows //= 2
    shape = (max(rows, 32),) + rest
    segments = int(max(2, min(2 ** rng.uniform(1, 13), shape[0] // 2)))
    if rng.random() < 0.5:
        dtype = [DataType.fp32, DataType.bf16][rng.integers(0, 2)]
        print(f"softmax and centering shape={shape} segments={segments} {dtype.name}", flush=True)
        RE.test_random_ragged_softmax_and_centering_against_numpy(stream, shape, segments, dtype)
    else:
        dtype = [DataType.fp32, DataType.bf16, DataType.fp16, DataType.fp8_e4m3, DataType.fp8_e5m2][rng.integers(0, 5)]
        print(f"broadcast shape={shape} segments={segments} {dtype.name}", flush=True)
        SB.test_broadcast_matches_a_loop_over_segments(stream, shape, segments, dtype)
    return ""


def rope_case(rng, stream):
    import test_expression_rope_gpu as RP
    head = int(rng.integers(1, 65)) * 2
    options = {}
    if rng.random() < 0.5:
        shape = (int(rng.integers(1, 4)), int(rng.integers(1, 6)), int(2 ** rng.uniform(0, 9)), head)
    else:
        shape = (int(rng.integers(1, 4)), int(2 ** rng.uniform(0, 9)), int(rng.integers(1, 6)), head)
        options.update(sequence_axis=1, head_dim_axis=3)
    if rng.random() < 0.4:
        options["rotary_dim"] = int(rng.integers(1, head // 2 + 1)) * 2
    if rng.random() < 0.4:
        options["interleaved"] = True
    if rng.random() < 0.3:
        options["inverse"] = True
    if rng.random() < 0.4:
        options["position_offset"] = int(rng.integers(0, 100))
    dtype = [DataType.fp32, DataType.fp16, DataType.bf16][rng.integers(0, 3)]
    print(f"{dtype.name} shape={shape} {options}", flush=True)
    RP.test_layouts_against_the_oracle(stream, shape, options, dtype)
    return ""


def backward_case(rng, stream):
    """Gradients of random polynomial graphs over broadcast operands (exact in fp32 on small integers), and of min / max reductions
    over rows of distinct values, against a reverse-mode walk in NumPy."""
    import test_expression_backward_gpu as B
    ex = ph.Expression
    rank = int(rng.integers(1, 4))
    left = 2 ** rng.uniform(0, 16)
    dims = []
    for d in range(rank):
        extent = int(max(1, round(left if d == rank - 1 else 2 ** rng.uniform(0, np.log2(max(left, 1.0001))))))
        dims.append(extent)
        left = max(left / extent, 1)
    total = int(np.prod(dims))

    def unbroadcast(g, shape):
        axes = tuple(a for a in range(len(shape)) if shape[a] == 1 and g.shape[a] != 1)
        return g.sum(axis=axes, keepdims=True) if axes else g

    if rng.random() < 0.3:
        # the gradient of a max / min over some axes goes to the one winner of every reduced group (distinct values: no ties)
        x = rng.permutation(total).reshape(dims).astype(np.int64) - total // 2
        if total >= (1 << 23):
            return ""
        axes = sorted(rng.choice(rank, int(rng.integers(1, rank + 1)), replace=False).tolist())
        scale = int(rng.choice([1, -1, 2]))
        kind = ["max", "min"][rng.integers(0, 2)]
        value = ex.input("x") * float(scale) + 1.0
        forward = value.reduce_max(axes) if kind == "max" else value.reduce_min(axes)
        seen = x * scale + 1
        best = (np.max if kind == "max" else np.min)(seen, axis=tuple(axes), keepdims=True)
        upstream = rng.integers(-3, 4, best.shape)
        want = {"x_grad": (seen == best) * upstream * scale}
        print(f"{kind}{axes} of x{dims} * {scale} + 1", flush=True)
        plan, got, _, _ = B.backward(forward, {"x": x.astype(np.float32), "e": upstream.astype(np.float32)}, stream, ["x"], upstream="e")
    else:
        names = "abc"[:int(rng.integers(2, 4))]
        values = {}
        nodes = []  # (expression, value, parents as (node index, function of the node's gradient -> the parent's share))
        for i, name in enumerate(names):
            shape = [e if i == 0 or rng.random() < 0.7 else 1 for e in dims]
            values[name] = rng.integers(-3, 4, shape).astype(np.int64)
            nodes.append((ex.input(name), values[name], [], 3))
        text = list(names)
        for _ in range(int(rng.integers(1, 5))):
            i, j = int(rng.integers(0, len(nodes))), int(rng.integers(0, len(nodes)))
            (x, xv, _, xb), (y, yv, _, yb) = nodes[i], nodes[j]
            op = ["add", "sub", "mul", "neg"][rng.integers(0, 4)]
            if op == "mul" and xb * yb > 60 or op in ("add", "sub") and xb + yb > 60:
                op = "neg"
            if op == "add":
                node = (x + y, xv + yv, [(i, lambda g: g), (j, lambda g: g)], xb + yb)
            elif op == "sub":
                node = (x - y, xv - yv, [(i, lambda g: g), (j, lambda g: -g)], xb + yb)
            elif op == "mul":
                node = (x * y, xv * yv, [(i, lambda g, yv=yv: g * yv), (j, lambda g, xv=xv: g * xv)], xb * yb)
            else:
                node = (-x, -xv, [(i, lambda g: -g)], xb)
            nodes.append(node)
            text.append(f"{op}({text[i]},{text[j]})" if op != "neg" else f"neg({text[i]})")
        for k, name in enumerate(names):  # every input takes part
            last = len(nodes) - 1
            x, xv, _, xb = nodes[last]
            y, yv, _, yb = nodes[k]
            nodes.append((x + y, xv + yv, [(last, lambda g: g), (k, lambda g: g)], xb + yb))
            text.append(f"add({text[last]},{name})")
        forward, out_value = nodes[-1][0], nodes[-1][1]
        out_shape = np.broadcast_shapes(*[values[n].shape for n in names])
        upstream = rng.integers(-2, 3, out_shape).astype(np.int64)
        grads = [None] * len(nodes)
        grads[-1] = upstream
        for index in range(len(nodes) - 1, -1, -1):
            if grads[index] is None:
                continue
            for parent, share in nodes[index][2]:
                g = unbroadcast(share(grads[index]), nodes[parent][1].shape)
                grads[parent] = g if grads[parent] is None else grads[parent] + g
        want = {name + "_grad": grads[k] for k, name in enumerate(names)}
        if max(int(np.abs(g).max()) for g in want.values()) >= (1 << 24):
            return ""
        print(f"dims={dims} shapes={[list(values[n].shape) for n in names]} {text[-1]}", flush=True)
        arrays = {n: values[n].astype(np.float32) for n in names}
        arrays["e"] = upstream.astype(np.float32)
        plan, got, _, _ = B.backward(forward, arrays, stream, list(names), upstream="e")
    for name, expected in want.items():
        assert got[name].shape == expected.shape, (name, got[name].shape, expected.shape)
        np.testing.assert_array_equal(got[name], expected.astype(np.float64), err_msg=f"{name} {plan.stage_descriptions()}")
    return " | ".join(plan.stage_kind_names())


FAMILIES = {"backward": backward_case, "ragged": ragged_case, "rope": rope_case, "views": views_case, "expressions": expressions_case, "conversions": conversions_case, "topk": topk_case, "topk_rows": topk_rows_case, "scans": scans_case, "reductions": reductions_case, "rows": rows_case}

if __name__ == "__main__":
    if len(sys.argv) != 4 or sys.argv[1] not in FAMILIES:
        sys.exit(__doc__)
    family, seed, cases = FAMILIES[sys.argv[1]], int(sys.argv[2]), int(sys.argv[3])
    rng = np.random.default_rng(seed)
    stream = ph.Stream(0)
    start = time.time()
    for case in range(cases):
        print(f"case {case}: ", end="", flush=True)
        variant = family(rng, stream)
        print(f"   ok {variant[:100]}  t={time.time() - start:.0f}s", flush=True)
    print(f"ALL OK: {cases} cases of {sys.argv[1]}, seed {seed}")
