"""Pins the CPU oracle's reductions (oracle/thor_oracle.c) against the reference's own known-answer vectors
(tests/golden/reduction_kats.json), numpy float64 closed forms and brute force on small shapes; and checks the host-side
geometry analysis (CubReduction::analyzeGeometry, no GPU needed) against the reference's geometry test table."""
import itertools
import json
import os

import numpy as np
import pytest

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
OPS = {"Sum": oracle.SUM, "Min": oracle.MIN, "Max": oracle.MAX, "Product": oracle.PRODUCT, "Mean": oracle.MEAN, "L1Norm": oracle.L1NORM,
       "L2Norm": oracle.L2NORM}


def kats():
    with open(os.path.join(GOLDEN, "reduction_kats.json")) as f:
        return json.load(f)


def as_f32(values):
    return np.array([np.nan if v is None else v for v in values], dtype=np.float32)


def view_of(case):
    base = as_f32(case["values"]).reshape(case["shape"])
    if "view_shape" in case:
        strides = [s * 4 for s in case["view_strides"]]
        return np.lib.stride_tricks.as_strided(base, shape=case["view_shape"], strides=strides), base
    return base, base


@pytest.mark.parametrize("case", kats()["value"], ids=lambda c: c["name"])
def test_value_kats(case):
    arr, _keep = view_of(case)
    for op_name, want in case["expect"].items():
        got = oracle.reduce(OPS[op_name], arr, oracle.FP32, case["axes"]).reshape(-1)
        np.testing.assert_allclose(got, np.array(want, dtype=np.float32), rtol=2e-6, atol=0)
        got64 = oracle.reduce_f64(OPS[op_name], arr, oracle.FP32, case["axes"]).reshape(-1)
        np.testing.assert_allclose(got64, np.array(want, dtype=np.float64), rtol=1e-12)


@pytest.mark.parametrize("case", kats()["arg"], ids=lambda c: c["name"])
def test_arg_kats(case):
    arr = as_f32(case["values"]).reshape(case["shape"])
    for name, op in (("argmin", oracle.ARGMIN), ("argmax", oracle.ARGMAX)):
        if name not in case:
            continue
        idx, val = oracle.arg_reduce(op, arr, oracle.FP32, case["axes"])
        assert idx.reshape(-1).tolist() == case[name]["index"]
        np.testing.assert_array_equal(val.reshape(-1), as_f32(case[name]["value"]))


def test_against_numpy_closed_forms_all_axis_subsets():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3, 4, 5, 6)).astype(np.float32)
    for k in range(1, 5):
        for axes in itertools.combinations(range(4), k):
            x64 = x.astype(np.float64)
            np.testing.assert_allclose(oracle.reduce_f64(oracle.SUM, x, oracle.FP32, axes), x64.sum(axis=axes, keepdims=True), rtol=1e-12)
            np.testing.assert_allclose(oracle.reduce(oracle.MEAN, x, oracle.FP32, axes), x64.mean(axis=axes, keepdims=True), rtol=1e-5, atol=1e-6)
            np.testing.assert_array_equal(oracle.reduce(oracle.MAX, x, oracle.FP32, axes), x.max(axis=axes, keepdims=True))
            np.testing.assert_array_equal(oracle.reduce(oracle.MIN, x, oracle.FP32, axes), x.min(axis=axes, keepdims=True))
            np.testing.assert_allclose(oracle.reduce(oracle.L2NORM, x, oracle.FP32, axes), np.sqrt((x64 ** 2).sum(axis=axes, keepdims=True)), rtol=1e-5)
            np.testing.assert_allclose(oracle.reduce(oracle.L1NORM, x, oracle.FP32, axes), np.abs(x64).sum(axis=axes, keepdims=True), rtol=1e-5)
            if np.prod([x.shape[a] for a in axes]) <= 30:  # longer products underflow fp32
                np.testing.assert_allclose(oracle.reduce(oracle.PRODUCT, x, oracle.FP32, axes), x64.prod(axis=axes, keepdims=True), rtol=1e-4)
            # argmax over the flattened reduced axes, lowest index on ties (no ties in continuous data)
            moved = np.moveaxis(x, axes, range(4 - k, 4)).reshape([x.shape[a] for a in range(4) if a not in axes] + [-1])
            idx, val = oracle.arg_reduce(oracle.ARGMAX, x, oracle.FP32, axes)
            np.testing.assert_array_equal(idx.reshape(moved.shape[:-1]), moved.argmax(axis=-1))
            np.testing.assert_array_equal(val.reshape(moved.shape[:-1]), moved.max(axis=-1))


def test_nan_propagation_scale_and_low_precision_io():
    x = np.array([[1.0, np.nan, 3.0], [4.0, 5.0, 6.0]], dtype=np.float32)
    assert np.isnan(oracle.reduce(oracle.MAX, x, oracle.FP32, [1]).reshape(-1)[0])
    assert np.isnan(oracle.reduce(oracle.MIN, x, oracle.FP32, [1]).reshape(-1)[0])
    assert oracle.reduce(oracle.MAX, x, oracle.FP32, [1]).reshape(-1)[1] == 6.0
    y = np.array([[1.0, 2.0, 3.0, 4.0]], dtype=np.float32)
    assert oracle.reduce(oracle.SUM, y, oracle.FP32, [1], scale=0.5).reshape(-1)[0] == 5.0
    # fp16 / bf16 inputs accumulate in fp32; outputs round once; fp8 saturates (reference KAT: 448 / 57344)
    h = np.full((1, 4096), 1.0, dtype=np.float16)
    assert oracle.reduce(oracle.SUM, h, oracle.FP16, [1], out_dtype=oracle.FP32).reshape(-1)[0] == 4096.0
    big = np.full((1, 8), 1000.0, dtype=np.float32)
    assert oracle.to_f32(oracle.reduce(oracle.SUM, big, oracle.FP32, [1], out_dtype=oracle.FP8_E4M3), oracle.FP8_E4M3).reshape(-1)[0] == 448.0
    big = np.full((1, 8), 30000.0, dtype=np.float32)
    assert oracle.to_f32(oracle.reduce(oracle.SUM, big, oracle.FP32, [1], out_dtype=oracle.FP8_E5M2), oracle.FP8_E5M2).reshape(-1)[0] == 57344.0


# ---- host-side geometry analysis of the product (pure host logic, runs without a GPU) -----------------------------------
@pytest.mark.parametrize("case", kats()["geometry"], ids=lambda c: f"{c['dims']}-{c['axes']}")
def test_geometry_table(case):
    from thor_amd import physical as ph
    g = ph.analyze_geometry(case["dims"], case["axes"])
    assert g.path == case["path"]
    assert bool(g.reduced_axes_are_contiguous) == case["contig"]
    assert (g.outer_size, g.reduction_size, g.inner_size, g.output_elements) == (case["outer"], case["R"], case["inner"], case["outputs"])
    assert list(g.output_dimensions[: g.rank]) == case["out_dims"]
    if "squeezed" in case:
        assert list(g.squeezed_output_dimensions[: g.squeezed_rank]) == case["squeezed"]
    for out_index, red_index, physical in case.get("map", []):
        assert ph.map_logical_reduction_index(case["dims"], case["axes"], out_index, red_index) == physical


@pytest.mark.parametrize("case", kats()["geometry_invalid"], ids=lambda c: f"{c['dims']}-{c['axes']}")
def test_geometry_rejects_invalid(case):
    from thor_amd import physical as ph
    with pytest.raises(ValueError):  # std::invalid_argument
        ph.analyze_geometry(case["dims"], case["axes"])


def test_geometry_index_map_is_a_bijection_in_row_major_order():
    from thor_amd import physical as ph
    for dims, axes in [([2], [0]), ([2, 3], [0]), ([2, 3], [1]), ([2, 3, 4], [0, 2]), ([3, 2, 2, 3], [1, 2]), ([2, 3, 4, 2], [0, 3])]:
        g = ph.analyze_geometry(dims, axes)
        seen = set()
        idx = np.arange(int(np.prod(dims))).reshape(dims)
        kept = [a for a in range(len(dims)) if a not in axes]
        moved = np.transpose(idx, kept + list(axes)).reshape(g.output_elements, g.reduction_size)
        for o in range(g.output_elements):
            for r in range(g.reduction_size):
                p = ph.map_logical_reduction_index(dims, axes, o, r)
                assert p == moved[o, r]
                seen.add(p)
        assert len(seen) == g.input_elements


def test_geometry_views_and_affine_rank1():
    from thor_amd import physical as ph
    assert ph.analyze_geometry([4, 5], [1], strides=[5, 1]).path == ph.CubReductionPath.ContiguousFixedSegment
    assert ph.analyze_geometry([5, 4], [1], strides=[1, 5]).path == ph.CubReductionPath.StridedFixedSegment
    diag = ph.analyze_geometry([4], [0], strides=[5])
    assert diag.path == ph.CubReductionPath.DeviceTransformReduce and diag.device_transform_uses_affine_stride and diag.affine_input_stride == 5


def test_generated_reduction_kernels_compile_for_gfx950():
    """Every kernel family is generated and cross-compiled with hipRTC on a host without a GPU."""
    import ctypes

    from thor_amd import _lib
    from thor_amd import physical as ph
    from thor_amd.dtypes import DataType
    L = _lib.load()
    cases = [(False, 0, DataType.fp32, DataType.fp32, [8192, 8192], [0, 1]), (False, 2, DataType.fp32, DataType.fp32, [8192, 8192], [1]),
             (True, 1, DataType.fp32, DataType.fp32, [8192, 8192], [1]), (False, 0, DataType.fp16, DataType.fp32, [64, 256, 56, 56], [0, 2, 3]),
             (False, 4, DataType.bf16, DataType.fp16, [32768, 1024], [0]), (True, 0, DataType.fp8_e4m3, DataType.fp16, [4, 3, 5], [1]),
             (False, 6, DataType.fp32, DataType.fp32, [4, 1 << 22], [1])]
    for is_arg, op, idt, odt, dims, axes in cases:
        src = ph.reduction_source(is_arg, op, idt, odt, dims, axes)
        assert "thor_reduce_main" in src
        code, size = ctypes.c_void_p(), ctypes.c_size_t()
        log = ctypes.create_string_buffer(1 << 14)
        opts = (ctypes.c_char_p * 1)(b"-ffp-contract=off")
        rc = L.thorhip_compile(src.encode(), b"reduce.hip", b"gfx950", opts, 1, ctypes.byref(code), ctypes.byref(size), log, 1 << 14)
        assert rc == 0, L.thorhip_last_error().decode()[:2000]
        L.thorhip_code_free(code)
