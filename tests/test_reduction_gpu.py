"""GPU parity of CubReduction / CubArgReduction against the reference's known-answer vectors and the CPU oracle."""
import json
import os

import numpy as np
import pytest

import oracle
from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, f32_to_gpu, from_storage, gpu_tensor, gpu_to_f32, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
OPS = {"Sum": (ph.CubReductionOp.Sum, oracle.SUM), "Min": (ph.CubReductionOp.Min, oracle.MIN), "Max": (ph.CubReductionOp.Max, oracle.MAX),
       "Product": (ph.CubReductionOp.Product, oracle.PRODUCT), "Mean": (ph.CubReductionOp.Mean, oracle.MEAN),
       "L1Norm": (ph.CubReductionOp.L1Norm, oracle.L1NORM), "L2Norm": (ph.CubReductionOp.L2Norm, oracle.L2NORM)}


def kats():
    with open(os.path.join(GOLDEN, "reduction_kats.json")) as f:
        return json.load(f)


def as_f32(values):
    return np.array([np.nan if v is None else v for v in values], dtype=np.float32)


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


@pytest.mark.parametrize("case", kats()["value"], ids=lambda c: c["name"])
def test_value_kats(stream, case):
    t = f32_to_gpu(as_f32(case["values"]).reshape(case["shape"]), DataType.fp32, stream)
    if "view_shape" in case:
        t = t.alias_view(case["view_shape"], case["view_strides"])
    for op_name, want in case["expect"].items():
        stamped = ph.CubReduction(OPS[op_name][0], case["axes"], DataType.fp32).stamp(t, stream)
        if case["path"] is not None:
            assert stamped.get_path() == case["path"]
        stamped.run()
        got = gpu_to_f32(stamped.get_output_tensor(), stream).reshape(-1)
        np.testing.assert_allclose(got, np.array(want, dtype=np.float32), rtol=2e-6, atol=0, err_msg=f"{case['name']} {op_name}")


@pytest.mark.parametrize("case", kats()["arg"], ids=lambda c: c["name"])
def test_arg_kats(stream, case):
    t = f32_to_gpu(as_f32(case["values"]).reshape(case["shape"]), DataType.fp32, stream)
    for name, op in (("argmin", ph.CubArgReductionOp.ArgMin), ("argmax", ph.CubArgReductionOp.ArgMax)):
        if name not in case:
            continue
        stamped = ph.CubArgReduction(op, case["axes"], value_output_dtype=DataType.fp32).stamp(t, stream)
        assert stamped.get_path() == case["path"]
        stamped.run()
        idx = copy_gpu_to_numpy(stamped.get_index_output_tensor(), stream).reshape(-1)
        val = gpu_to_f32(stamped.get_value_output_tensor(), stream).reshape(-1)
        assert idx.dtype == np.uint32 and idx.tolist() == case[name]["index"], f"{case['name']} {name}"
        np.testing.assert_array_equal(val, as_f32(case[name]["value"]))


SHAPES = [
    ([1], [0]), ([7], [0]), ([1000], [0]), ([4099], [0]), ([1 << 20], [0]), ((1 << 20) + 3, None),
    ([3, 5], [1]), ([64, 1], [1]), ([33, 17], [1]), ([128, 64], [1]), ([100, 1000], [1]), ([7, 4096], [1]), ([5, 8191], [1]), ([3, 70000], [1]),
    ([2, 1 << 19], [1]), ([1000, 3], [0]), ([64, 64], [0]), ([4097, 8], [0]), ([2, 300, 40], [1]), ([5, 6, 7, 8], [1, 2]), ([5, 6, 7, 8], [0, 1]),
    ([4, 6, 10, 12], [0, 2, 3]), ([3, 4, 5, 6], [1, 3]), ([2, 3, 4, 5, 2], [0, 2, 4]), ([8, 16, 32], [0, 2]),
    # rows no vector divides: vectors at addresses aligned to the element only, the rest of the row one by one
    ([100, 1001], [1]), ([37, 50257], [1]), ([5000, 63], [1]), ([3, 70001], [1]), ([9, 131], [1]),
    # a middle axis over an inner extent of a few elements: the rows kernel with one accumulator per inner element
    ([64, 300, 4], [1]), ([4096, 50, 2], [1]), ([33, 1000, 4], [1]), ([7, 5, 2, 2], [1]), ([2000, 6, 4], [1]),
    # columns over an inner extent no vector divides: the last vector ends with the extent and overlaps the one before it
    ([300, 1001], [0]), ([5000, 63], [0]), ([17, 50257], [0]), ([3, 200, 77], [1]), ([40, 9, 131], [0, 1]), ([2, 1000, 17], [1]), ([600, 9], [0]),
]


# One shape per kernel family the planner can choose (whole tensor short and long, rows by lanes / by a block / split, columns,
# columns split, disjoint axes, rows and columns no vector divides, interleaved outputs): these run all seven operations.  The
# operations differ in the accumulate / finalise functor only, so the other shapes run a sum and a selection; every shape runs in
# fp32 and in one 16-bit dtype (fp16 and bf16 alternate down the list).
ALL_OPS_SHAPES = {((4099,), (0,)), ((1 << 20,), (0,)), ((100, 1000), (1,)), ((3, 70000), (1,)), ((2, 1 << 19), (1,)), ((64, 64), (0,)), ((4097, 8), (0,)),
                  ((4, 6, 10, 12), (0, 2, 3)), ((37, 50257), (1,)), ((64, 300, 4), (1,)), ((300, 1001), (0,)), ((3, 200, 77), (1,)), ((3, 5), (1,))}
VALUE_CASES = []
for _i, (_d, _a) in enumerate((d, a) for d, a in SHAPES if a is not None):
    VALUE_CASES += [(_d, _a, DataType.fp32), (_d, _a, DataType.fp16 if _i % 2 == 0 else DataType.bf16)]


@pytest.mark.parametrize("dims,axes,dtype", VALUE_CASES, ids=lambda v: v.name if isinstance(v, DataType) else str(v))
def test_value_ops_against_oracle(stream, dims, axes, dtype):
    rng = np.random.default_rng(abs(hash((tuple(dims), tuple(axes)))) % (1 << 31))
    x = to_storage(rng.standard_normal(dims).astype(np.float32), dtype)
    t = copy_numpy_to_gpu(x, stream, dtype)
    reduction_size = int(np.prod([dims[a] for a in axes]))
    every_op = dtype == DataType.fp32 and (tuple(dims), tuple(axes)) in ALL_OPS_SHAPES
    for op_name, (op, oop) in OPS.items():
        if op_name == "Product" and reduction_size > 64:
            continue
        if not every_op and op_name not in (("Sum", "Max") if dtype == DataType.fp32 else ("Mean", "Min")):
            continue
        stamped = ph.CubReduction(op, axes, DataType.fp32).stamp(t, stream)
        stamped.run()
        got = gpu_to_f32(stamped.get_output_tensor(), stream)
        exact = oracle.reduce_f64(oop, x, int(dtype), axes)
        if op_name in ("Min", "Max"):
            np.testing.assert_array_equal(got, exact.astype(np.float32), err_msg=op_name)
        else:
            # fp32 accumulation in a different order than the oracle: 1e-5 relative to the magnitude that was summed
            magnitude = oracle.reduce_f64(oracle.L1NORM, x, int(dtype), axes) if op_name in ("Sum", "Mean") else np.abs(exact)
            if op_name == "Mean":
                magnitude = magnitude / reduction_size
            tol = 1e-5 * np.maximum(magnitude, np.abs(exact)) + 1e-30
            assert np.all(np.abs(got.astype(np.float64) - exact) <= tol), f"{op_name} {stamped.get_kernel_variant()}"


@pytest.mark.parametrize("dims,axes", [(d, a) for d, a in SHAPES if a is not None], ids=lambda v: str(v))
def test_arg_ops_against_oracle_with_ties_and_nans(stream, dims, axes):
    rng = np.random.default_rng(7)
    # few distinct values -> many ties; sprinkle NaNs and infinities
    x = rng.integers(-3, 4, size=dims).astype(np.float32)
    flat = x.reshape(-1)
    if flat.size > 10:
        flat[rng.integers(0, flat.size, size=max(1, flat.size // 50))] = np.nan
        flat[rng.integers(0, flat.size, size=max(1, flat.size // 50))] = np.inf
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    # both index widths for the shapes that stand for a kernel family; elsewhere arg-min writes UINT32 and arg-max UINT64
    both_widths = (tuple(dims), tuple(axes)) in ALL_OPS_SHAPES
    for op, oop in ((ph.CubArgReductionOp.ArgMin, oracle.ARGMIN), (ph.CubArgReductionOp.ArgMax, oracle.ARGMAX)):
        for index_dtype in (DataType.uint32, DataType.uint64):
            if not both_widths and (index_dtype == DataType.uint64) != (op == ph.CubArgReductionOp.ArgMax):
                continue
            stamped = ph.CubArgReduction(op, axes, value_output_dtype=DataType.fp32, index_output_dtype=index_dtype).stamp(t, stream)
            stamped.run()
            idx = copy_gpu_to_numpy(stamped.get_index_output_tensor(), stream)
            val = gpu_to_f32(stamped.get_value_output_tensor(), stream)
            want_idx, want_val = oracle.arg_reduce(oop, x, oracle.FP32, axes)
            np.testing.assert_array_equal(idx.astype(np.uint64), want_idx)
            np.testing.assert_array_equal(val, want_val)


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16], ids=lambda d: d.name)
def test_rows_no_vector_divides_and_rows_that_begin_off_a_vector(stream, dtype):
    rng = np.random.default_rng(3)
    x = to_storage(rng.standard_normal((64, 1003)).astype(np.float32), dtype)
    t = copy_numpy_to_gpu(x, stream, dtype)
    stamped = ph.CubReduction(ph.CubReductionOp.Sum, [1], DataType.fp32).stamp(t, stream)
    assert "unaligned_vectors" in stamped.get_kernel_variant()
    stamped.run()
    exact = oracle.reduce_f64(oracle.SUM, x, int(dtype), [1])
    magnitude = oracle.reduce_f64(oracle.L1NORM, x, int(dtype), [1])
    assert np.all(np.abs(gpu_to_f32(stamped.get_output_tensor(), stream).astype(np.float64) - exact) <= 1e-5 * magnitude + 1e-30)
    # a view whose rows have a vector's length but begin one element into the storage
    for rows_in_view, row_stride in ((60, 1003), (64000 // 1000, 1000)):
        view = t.alias_view([rows_in_view, 1000], [row_stride, 1], element_offset=1)
        stamped = ph.CubReduction(ph.CubReductionOp.Max, [1], DataType.fp32).stamp(view, stream)
        stamped.run()
        carrier = x.reshape(-1)[1:]
        rows = np.stack([carrier[r * row_stride:r * row_stride + 1000] for r in range(rows_in_view)])
        np.testing.assert_array_equal(gpu_to_f32(stamped.get_output_tensor(), stream), oracle.reduce_f64(oracle.MAX, rows, int(dtype), [1]).astype(np.float32),
                                      err_msg=stamped.get_kernel_variant())


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.bf16], ids=lambda d: d.name)
def test_columns_over_inner_extents_no_vector_divides(stream, dtype):
    """Lanes own whole vectors of outputs although the inner extent is odd; every output is stored once, by one owner: small
    integers make the sums exact, so an output summed twice or taken from a neighbour shows.  Split and unsplit shapes, an
    outer axis, the arg form, and a view that begins one element into the storage."""
    rng = np.random.default_rng(11)
    for dims, axes in (([3000, 1001], [0]), ([40, 50257], [0]), ([5, 700, 77], [1]), ([100000, 19], [0])):
        x = to_storage(rng.integers(-4, 5, size=dims).astype(np.float32), dtype)
        t = copy_numpy_to_gpu(x, stream, dtype)
        stamped = ph.CubReduction(ph.CubReductionOp.Sum, axes, DataType.fp32).stamp(t, stream)
        assert "columns(" in stamped.get_kernel_variant() and "unaligned_vectors" in stamped.get_kernel_variant(), stamped.get_kernel_variant()
        stamped.run()
        want = oracle.reduce_f64(oracle.SUM, x, int(dtype), axes).astype(np.float32)
        np.testing.assert_array_equal(gpu_to_f32(stamped.get_output_tensor(), stream).reshape(want.shape), want, err_msg=stamped.get_kernel_variant())
        arg = ph.CubArgReduction(ph.CubArgReductionOp.ArgMax, axes, value_output_dtype=DataType.fp32, index_output_dtype=DataType.uint32).stamp(t, stream)
        arg.run()
        want_idx, want_val = oracle.arg_reduce(oracle.ARGMAX, x, int(dtype), axes)
        np.testing.assert_array_equal(copy_gpu_to_numpy(arg.get_index_output_tensor(), stream).astype(np.uint64).reshape(want_idx.shape), want_idx,
                                      err_msg=arg.get_kernel_variant())
        np.testing.assert_array_equal(gpu_to_f32(arg.get_value_output_tensor(), stream).reshape(want_val.shape), want_val)
    # an even inner extent read from one element into the storage: no address is a multiple of the vector
    x = to_storage(rng.integers(-4, 5, size=(500 * 1000 + 8,)).astype(np.float32), dtype)
    t = copy_numpy_to_gpu(x, stream, dtype)
    view = t.alias_view([500, 1000], [1000, 1], element_offset=1)
    stamped = ph.CubReduction(ph.CubReductionOp.Sum, [0], DataType.fp32).stamp(view, stream)
    stamped.run()
    want = oracle.reduce_f64(oracle.SUM, x[1:1 + 500 * 1000].reshape(500, 1000), int(dtype), [0]).astype(np.float32)
    np.testing.assert_array_equal(gpu_to_f32(stamped.get_output_tensor(), stream).reshape(want.shape), want, err_msg=stamped.get_kernel_variant())


def test_small_inner_extents_take_the_rows_kernel_with_interleaved_outputs(stream):
    x = np.arange(64 * 300 * 4, dtype=np.float32).reshape(64, 300, 4) % 17
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    stamped = ph.CubReduction(ph.CubReductionOp.Sum, [1], DataType.fp32).stamp(t, stream)
    assert "outputs_per_row=4" in stamped.get_kernel_variant(), stamped.get_kernel_variant()
    stamped.run()
    np.testing.assert_array_equal(gpu_to_f32(stamped.get_output_tensor(), stream).reshape(64, 4), x.sum(axis=1))  # small integers: exact
    arg = ph.CubArgReduction(ph.CubArgReductionOp.ArgMax, [1], value_output_dtype=DataType.fp32, index_output_dtype=DataType.uint32).stamp(t, stream)
    assert "outputs_per_row=4" in arg.get_kernel_variant(), arg.get_kernel_variant()
    arg.run()
    np.testing.assert_array_equal(copy_gpu_to_numpy(arg.get_index_output_tensor(), stream).reshape(64, 4), x.argmax(axis=1).astype(np.uint32))
    np.testing.assert_array_equal(gpu_to_f32(arg.get_value_output_tensor(), stream).reshape(64, 4), x.max(axis=1))


def test_output_dtypes_scale_and_fp8_saturation(stream):
    x = np.full((2, 8), 1000.0, dtype=np.float32)
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    # reference KAT: sums far above the fp8 range saturate to 448 / 57344 (CubReductionDTypeAndLifecycleTest.cpp:205-222)
    for dt, sat in ((DataType.fp8_e4m3, 448.0), (DataType.fp8_e5m2, 57344.0)):
        big = copy_numpy_to_gpu(np.full((2, 8), 30000.0, dtype=np.float32), stream, DataType.fp32)
        s = ph.CubReduction(ph.CubReductionOp.Sum, 1, dt).stamp(big, stream)
        s.run()
        assert gpu_to_f32(s.get_output_tensor(), stream).reshape(-1).tolist() == [sat, sat]
    for dt in (DataType.fp16, DataType.bf16, DataType.fp32):
        s = ph.CubReduction(ph.CubReductionOp.Sum, 1, dt, output_scale=0.25).stamp(t, stream)
        s.run()
        assert gpu_to_f32(s.get_output_tensor(), stream).reshape(-1).tolist() == [2000.0, 2000.0]
        s.run(output_scale=0.5)
        assert gpu_to_f32(s.get_output_tensor(), stream).reshape(-1).tolist() == [4000.0, 4000.0]
    # default output dtype = input dtype
    h = copy_numpy_to_gpu(to_storage(np.ones((3, 5), np.float32), DataType.bf16), stream, DataType.bf16)
    s = ph.CubReduction(ph.CubReductionOp.Sum, 1).stamp(h, stream)
    assert s.get_output_tensor().get_data_type() == DataType.bf16
    s.run()
    assert gpu_to_f32(s.get_output_tensor(), stream).reshape(-1).tolist() == [5.0, 5.0, 5.0]


def test_nan_and_inf_propagation(stream):
    x = np.array([[1.0, np.nan, 3.0, 2.0], [np.inf, 1.0, -np.inf, 0.0], [1.0, 2.0, 3.0, 4.0]], dtype=np.float32)
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    mx = ph.CubReduction(ph.CubReductionOp.Max, 1, DataType.fp32).stamp(t, stream)
    mn = ph.CubReduction(ph.CubReductionOp.Min, 1, DataType.fp32).stamp(t, stream)
    sm = ph.CubReduction(ph.CubReductionOp.Sum, 1, DataType.fp32).stamp(t, stream)
    for s in (mx, mn, sm):
        s.run()
    a, b, c = (gpu_to_f32(s.get_output_tensor(), stream).reshape(-1) for s in (mx, mn, sm))
    assert np.isnan(a[0]) and a[1] == np.inf and a[2] == 4.0
    assert np.isnan(b[0]) and b[1] == -np.inf and b[2] == 1.0
    assert np.isnan(c[0]) and np.isnan(c[1]) and c[2] == 10.0


def test_repeated_runs_are_bit_identical_and_preallocated_output(stream):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1 << 20) + 77).astype(np.float32)
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    out = gpu_tensor([1], DataType.fp32)
    s = ph.CubReduction(ph.CubReductionOp.Sum, 0, DataType.fp32).stamp(t, stream, preallocated_output=out)
    assert s.get_output_tensor().mem_ptr() == out.mem_ptr()
    results = []
    for _ in range(5):
        s.run()
        results.append(copy_gpu_to_numpy(out, stream).view(np.uint32)[0])
    assert len(set(results)) == 1
    with pytest.raises(ValueError):
        ph.CubReduction(ph.CubReductionOp.Sum, 0, DataType.fp32).stamp(t, stream, preallocated_output=gpu_tensor([3], DataType.fp32))
    with pytest.raises(ValueError):
        ph.CubReduction(ph.CubReductionOp.Sum, 5, DataType.fp32).stamp(t, stream)
    with pytest.raises(ValueError):
        ph.CubReduction(ph.CubReductionOp.Sum, 0).stamp(copy_numpy_to_gpu(np.arange(4, dtype=np.int32), stream, DataType.int32), stream)


def test_views_diagonal_and_broadcast_alias(stream):
    x = np.arange(25, dtype=np.float32).reshape(5, 5)
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    diag = t.alias_view([5], [6])
    s = ph.CubReduction(ph.CubReductionOp.Sum, 0, DataType.fp32).stamp(diag, stream)
    assert s.get_path() == ph.CubReductionPath.DeviceTransformReduce
    s.run()
    assert gpu_to_f32(s.get_output_tensor(), stream).reshape(-1)[0] == np.trace(x)
    tr = t.alias_view([5, 5], [1, 5])  # transposed view: row sums of the view are column sums of x
    s = ph.CubReduction(ph.CubReductionOp.Sum, 1, DataType.fp32).stamp(tr, stream)
    s.run()
    np.testing.assert_array_equal(gpu_to_f32(s.get_output_tensor(), stream).reshape(-1), x.sum(axis=0))
    amax = ph.CubArgReduction(ph.CubArgReductionOp.ArgMax, 1, value_output_dtype=DataType.fp32).stamp(tr, stream)
    amax.run()
    assert copy_gpu_to_numpy(amax.get_index_output_tensor(), stream).reshape(-1).tolist() == [4] * 5


PERMUTED = [
    # (storage shape, permutation giving the view, reduced view axes)
    ((96, 200), (1, 0), [1]),            # transposed matrix, reduce along the view's rows = the storage's columns
    ((40, 33, 64), (2, 0, 1), [1]),      # contiguous storage axis first in the view, reduce a middle storage axis
    ((40, 33, 64), (2, 0, 1), [1, 2]),   # ... and both other axes
    ((12, 16, 48), (0, 2, 1), [2]),      # batch kept, inner two swapped
    ((7, 130), (1, 0), [1]),             # lane axis not a multiple of the vector width
    # outputs whose fastest axis is not the lane axis: written through the LDS transpose
    ((37, 5, 132), (2, 1, 0), [1]),      # ragged tiles in both directions
    ((64, 8, 256), (2, 1, 0), [1]),
    ((20, 3, 17, 64), (3, 1, 0, 2), [1]),  # two kept axes after the lane axis
    ((300, 2, 16), (2, 1, 0), [1]),      # one vector-wide lane axis
]
TRANSPOSED_STORE = {((40, 33, 64), (2, 0, 1), (1,)), ((37, 5, 132), (2, 1, 0), (1,)), ((64, 8, 256), (2, 1, 0), (1,)), ((20, 3, 17, 64), (3, 1, 0, 2), (1,)),
                    ((300, 2, 16), (2, 1, 0), (1,))}


# fp32 over every view; fp16 (vectors twice as long) over the views whose outputs leave through the LDS transpose and one that does not
PERMUTED_CASES = [(s, p, a, DataType.fp32) for s, p, a in PERMUTED] + [(s, p, a, DataType.fp16) for s, p, a in PERMUTED
                                                                        if (s, p, tuple(a)) in TRANSPOSED_STORE or s == (7, 130)]


@pytest.mark.parametrize("shape,perm,axes,dtype", PERMUTED_CASES, ids=[f"{s}-{p}-{a}-{d.name}".replace(" ", "") for s, p, a, d in PERMUTED_CASES])
def test_permuted_views_reduce_with_lanes_on_the_contiguous_kept_axis(stream, shape, perm, axes, dtype):
    """Dense tensors seen through a permuted view (what Expression transposes hand to reductions): values and arg indices
    must equal those of the materialised permutation."""
    rng = np.random.default_rng(12)
    x = rng.integers(-8, 9, shape).astype(np.float32)  # small integers: sums are exact in any order
    storage = to_storage(x, dtype)
    t = copy_numpy_to_gpu(storage, stream, dtype)
    strides = [int(np.prod(shape[i + 1:])) for i in range(len(shape))]
    view = t.alias_view([shape[p] for p in perm], [strides[p] for p in perm])
    logical = np.ascontiguousarray(np.transpose(x, perm))
    for name in (("Sum", "Max", "L1Norm") if dtype == DataType.fp32 else ("Sum", "Min")):
        stamped = ph.CubReduction(OPS[name][0], axes, DataType.fp32).stamp(view, stream)
        stamped.run()
        want = oracle.reduce(OPS[name][1], logical, oracle.FP32, axes)
        np.testing.assert_array_equal(gpu_to_f32(stamped.get_output_tensor(), stream).reshape(want.shape), want, err_msg=f"{name} {stamped.get_kernel_variant()}")
    assert "view_columns" in stamped.get_kernel_variant()
    assert ("transposed_store" in stamped.get_kernel_variant()) == ((shape, perm, tuple(axes)) in TRANSPOSED_STORE), stamped.get_kernel_variant()
    for op, oracle_op in ((ph.CubArgReductionOp.ArgMax, oracle.ARGMAX), (ph.CubArgReductionOp.ArgMin, oracle.ARGMIN)):
        arg = ph.CubArgReduction(op, axes, value_output_dtype=DataType.fp32).stamp(view, stream)
        arg.run()
        want_index, want_value = oracle.arg_reduce(oracle_op, logical, oracle.FP32, axes)
        np.testing.assert_array_equal(copy_gpu_to_numpy(arg.get_index_output_tensor(), stream).reshape(want_index.shape).astype(np.uint64), want_index)
        np.testing.assert_array_equal(gpu_to_f32(arg.get_value_output_tensor(), stream).reshape(want_value.shape), want_value)


def test_config3_full_size_properties(stream):
    """BASELINE config 3, fp32 [8192, 8192] N(0,1): full sum, row sum, row max, row argmax.  Checked at full size against
    the float64 oracle (rows are independent, so the oracle finishes in seconds) and through invariants."""
    rng = np.random.default_rng(1236)
    x = rng.standard_normal((8192, 8192), dtype=np.float32)
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    full = ph.CubReduction(ph.CubReductionOp.Sum, [0, 1], DataType.fp32).stamp(t, stream)
    rows = ph.CubReduction(ph.CubReductionOp.Sum, 1, DataType.fp32).stamp(t, stream)
    rmax = ph.CubReduction(ph.CubReductionOp.Max, 1, DataType.fp32).stamp(t, stream)
    amax = ph.CubArgReduction(ph.CubArgReductionOp.ArgMax, 1, produce_value=False).stamp(t, stream)
    for s in (full, rows, rmax, amax):
        s.run()
    got_full = gpu_to_f32(full.get_output_tensor(), stream).reshape(-1)[0]
    got_rows = gpu_to_f32(rows.get_output_tensor(), stream).reshape(-1)
    got_max = gpu_to_f32(rmax.get_output_tensor(), stream).reshape(-1)
    got_arg = copy_gpu_to_numpy(amax.get_index_output_tensor(), stream).reshape(-1)
    exact_rows = x.astype(np.float64).sum(axis=1)
    abs_rows = np.abs(x).astype(np.float64).sum(axis=1)
    assert np.all(np.abs(got_rows - exact_rows) <= 1e-5 * np.maximum(np.abs(exact_rows), 1e-2 * abs_rows))
    assert abs(got_full - exact_rows.sum()) <= 1e-5 * max(abs(exact_rows.sum()), 1e-3 * abs_rows.sum())
    np.testing.assert_array_equal(got_max, x.max(axis=1))
    np.testing.assert_array_equal(got_arg, x.argmax(axis=1).astype(np.uint32))
    assert got_arg.dtype == np.uint32
    # invariants: the sum of the row sums equals the full sum; the value at the argmax is the row max
    assert abs(got_rows.astype(np.float64).sum() - got_full) <= 1e-5 * abs_rows.sum() * 1e-3 + 1e-5 * abs(got_full)
    np.testing.assert_array_equal(x[np.arange(8192), got_arg], got_max)


def test_split_reductions_whose_last_share_folds_agree_with_the_finishing_launch(stream, monkeypatch):
    """THOR_REDUCE_TICKETS=2 makes every split reduction fold inside its main launch (the share that arrives last does it); the
    default keeps a finishing launch for whole-tensor and column reductions.  Small integers: every order gives the same bits."""
    rng = np.random.default_rng(21)
    for dims, axes in (([8192, 1024], [0]), ([4096, 1001], [0]), ([3, 6000, 260], [1]), ([1 << 21], [0])):
        x = rng.integers(-4, 5, size=dims).astype(np.float32)
        t = copy_numpy_to_gpu(x, stream, DataType.fp32)
        results = {}
        for mode in ("0", "2"):
            monkeypatch.setenv("THOR_REDUCE_TICKETS", mode)
            stamped = ph.CubReduction(ph.CubReductionOp.Sum, axes, DataType.fp32).stamp(t, stream)
            assert ("last_share_folds" in stamped.get_kernel_variant()) == (mode == "2"), stamped.get_kernel_variant()
            for _ in range(2):  # the ticket words are left at zero for the next run
                stamped.run()
            arg = ph.CubArgReduction(ph.CubArgReductionOp.ArgMax, axes, value_output_dtype=DataType.fp32).stamp(t, stream)
            arg.run()
            results[mode] = (gpu_to_f32(stamped.get_output_tensor(), stream), copy_gpu_to_numpy(arg.get_index_output_tensor(), stream))
        want = oracle.reduce_f64(oracle.SUM, x, oracle.FP32, axes).astype(np.float32)
        np.testing.assert_array_equal(results["0"][0].reshape(want.shape), want)
        np.testing.assert_array_equal(results["2"][0].reshape(want.shape), want)
        want_idx, _ = oracle.arg_reduce(oracle.ARGMAX, x, oracle.FP32, axes)
        np.testing.assert_array_equal(results["0"][1].astype(np.uint64).reshape(want_idx.shape), want_idx)
        np.testing.assert_array_equal(results["2"][1].astype(np.uint64).reshape(want_idx.shape), want_idx)
