"""Expression::rotaryPositionEmbedding on the GPU against the oracle, the double-precision known answers, the properties of a
rotation at full size, and the reference's own test cases (bindings/python/test/core/physical/test_expression_attention.py:
4262-4400 forward parameterisations, :4577-4612 backward, :4660-4760 validation; ExpressionConvenienceOpsTest.cpp:3503-3700)."""
from __future__ import annotations

import json
import os

import numpy as np
import pytest

import oracle
from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, from_storage, to_storage
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex
from thor_amd.physical import RotaryScalingKind

pytestmark = pytest.mark.gpu

with open(os.path.join(os.path.dirname(__file__), "golden", "rope_kats.json")) as f:
    CASES = json.load(f)["cases"]
KIND = {k.name: k for k in RotaryScalingKind}
ORACLE_KIND = {RotaryScalingKind.none: oracle.ROPE_NONE, RotaryScalingKind.linear: oracle.ROPE_LINEAR, RotaryScalingKind.dynamic_ntk: oracle.ROPE_DYNAMIC_NTK,
               RotaryScalingKind.yarn: oracle.ROPE_YARN, RotaryScalingKind.longrope: oracle.ROPE_LONGROPE, RotaryScalingKind.llama3: oracle.ROPE_LLAMA3}
EPS32 = float(np.finfo(np.float32).eps)
# one unit in the last place of the storage type at the magnitudes the tests use (|y| < 8)
STORAGE_ULP = {DataType.fp32: 0.0, DataType.fp16: 2.0 ** -8, DataType.bf16: 2.0 ** -5, DataType.fp8_e4m3: 0.5, DataType.fp8_e5m2: 1.0}


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def run(outputs, inputs, stream):
    plan = ex.compile(ex.outputs(outputs), device_num=0).stamp(inputs, stream)
    plan.run()
    return plan


def oracle_rope(carrier, dtype, options, position_ids=None, effective_sequence_length=None, out_dtype=None):
    kw = dict(options)
    kw["scaling_kind"] = ORACLE_KIND[kw.get("scaling_kind", RotaryScalingKind.none)]
    kw.pop("output_dtype", None)
    return oracle.rope(carrier, int(dtype), position_ids=position_ids, effective_sequence_length=effective_sequence_length,
                       out_dtype=None if out_dtype is None else int(out_dtype), **kw)


def angle_tolerance(x32, max_position, dtype, factor=1.0):
    """Device powf / sinf / cosf stay within 2 ulp of the correctly rounded ones the oracle uses; an angle t = p * f off by a few
    ulp moves the rotated pair by |pair| * dt, which grows with the position.  Plus one storage rounding."""
    largest = float(np.abs(x32).max()) * factor
    return 1.5 * largest * (8 * EPS32 * max(max_position, 1.0) + 8 * EPS32) + STORAGE_ULP[dtype]


def options_of(case):
    o = dict(case["options"])
    if "scaling_kind" in o:
        o["scaling_kind"] = KIND[o["scaling_kind"]]
    return o


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_known_answers_and_oracle(stream, case, dtype):
    o = options_of(case)
    shape = case["shape"]
    x = to_storage(np.array(case["x"], np.float32).reshape(shape), dtype)
    inputs = {"x": copy_numpy_to_gpu(x, stream, dtype)}
    ids = length = None
    if case["position_ids"] is not None:
        ids = ex.input("positions")
        inputs["positions"] = copy_numpy_to_gpu(np.array(case["position_ids"], np.uint32), stream, DataType.uint32)
    if case["effective_sequence_length"] is not None:
        length = ex.input("length")
        inputs["length"] = copy_numpy_to_gpu(np.array([case["effective_sequence_length"]], np.uint32), stream, DataType.uint32)
    plan = run({"y": ex.input("x").rope(position_ids=ids, effective_sequence_length=length, **o)}, inputs, stream)
    assert plan.output("y").get_dimensions() == shape and plan.output("y").get_data_type() == dtype
    assert plan.stage_kind_names()[-1] == "FusedKernel"
    got = from_storage(copy_gpu_to_numpy(plan.output("y"), stream), dtype).astype(np.float64)
    positions = case["position_ids"] if case["position_ids"] is not None else [shape[o.get("sequence_axis", 2)] + o.get("position_offset", 0)]
    tol = angle_tolerance(np.array(case["x"], np.float32), float(max(positions)), dtype, 1.5)
    want = from_storage(oracle_rope(x, dtype, o, case["position_ids"], case["effective_sequence_length"]), dtype).astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=0, atol=tol)
    np.testing.assert_allclose(got, np.array(case["expected"]).reshape(shape), rtol=0, atol=tol + 4e-6 + STORAGE_ULP[dtype])


LAYOUTS = [
    ((2, 8, 512, 128), {}),
    ((2, 8, 512, 128), {"interleaved": True, "position_offset": 100}),
    ((2, 8, 300, 128), {"rotary_dim": 96}),
    ((2, 8, 300, 128), {"rotary_dim": 64, "interleaved": True, "inverse": True}),
    ((4, 300, 6, 64), {"sequence_axis": 1, "head_dim_axis": 3}),
    ((1000, 12, 64), {"sequence_axis": 0, "head_dim_axis": 2, "rotary_dim": 32}),
    ((3, 5, 70, 36), {"rotary_dim": 20}),                                      # vectors narrower than 16 bytes
    ((3, 5, 70, 30), {"interleaved": True}),
    ((2, 24, 5, 33), {"sequence_axis": 3, "head_dim_axis": 1}),                # the head dimension is not the last axis
    ((1, 1, 1, 2), {}),                                                        # one pair at position 0: the identity
    ((2, 3, 1, 6), {"rotary_dim": 2, "position_offset": 9}),
    ((2, 3, 5, 6), {"rotary_dim": 2, "interleaved": True}),
    ((7, 2), {"sequence_axis": 0, "head_dim_axis": 1}),                        # rank 2
    ((3, 4, 2, 5, 16), {"sequence_axis": 1, "head_dim_axis": 4}),              # two axes between sequence and head dimension
    ((6, 40, 16), {"sequence_axis": 1, "head_dim_axis": 2, "scaling_kind": RotaryScalingKind.llama3, "scaling_factor": 8.0,
                   "original_max_position_embeddings": 16, "base": 500000.0}),
    ((2, 4, 200, 64), {"scaling_kind": RotaryScalingKind.yarn, "scaling_factor": 4.0, "original_max_position_embeddings": 64}),
    ((2, 4, 200, 64), {"scaling_kind": RotaryScalingKind.dynamic_ntk, "scaling_factor": 2.0, "original_max_position_embeddings": 64}),
    ((2, 4, 200, 64), {"scaling_kind": RotaryScalingKind.linear, "scaling_factor": 4.0}),
    # halves that are not whole 64-byte sectors: two adjacent lanes share the pairs
    ((2, 3, 50, 80), {}), ((2, 3, 33, 96), {"position_offset": 4}), ((3, 2, 40, 128), {"rotary_dim": 80}), ((2, 2, 17, 48), {"inverse": True}),
    ((2, 50, 3, 80), {"sequence_axis": 1, "head_dim_axis": 3}), ((2, 19, 6, 96), {"sequence_axis": 1, "head_dim_axis": 3, "rotary_dim": 80}),
]


def layout_id(shape, options):
    return "x".join(str(d) for d in shape) + "".join("-" + k + "=" + str(getattr(v, "name", v)) for k, v in options.items())


@pytest.mark.parametrize("dtype", [DataType.fp32, DataType.fp16, DataType.bf16], ids=lambda d: d.name)
@pytest.mark.parametrize("shape,options", LAYOUTS, ids=[layout_id(s, o) for s, o in LAYOUTS])
def test_layouts_against_the_oracle(stream, shape, options, dtype):
    rng = np.random.default_rng(31)
    x32 = rng.standard_normal(shape).astype(np.float32)
    x = to_storage(x32, dtype)
    plan = run({"y": ex.input("x").rope(**options)}, {"x": copy_numpy_to_gpu(x, stream, dtype)}, stream)
    got = from_storage(copy_gpu_to_numpy(plan.output("y"), stream), dtype).astype(np.float64)
    want = from_storage(oracle_rope(x, dtype, options), dtype).astype(np.float64)
    seq = shape[options.get("sequence_axis", 2)] + options.get("position_offset", 0)
    np.testing.assert_allclose(got, want, rtol=0, atol=angle_tolerance(x32, seq, dtype))
    # beyond the rotary part nothing changes, bit for bit
    rotary = options.get("rotary_dim", 0)
    if rotary:
        tail = [slice(None)] * len(shape)
        tail[options.get("head_dim_axis", 3)] = slice(rotary, None)
        assert np.array_equal(copy_gpu_to_numpy(plan.output("y"), stream)[tuple(tail)], x[tuple(tail)])


@pytest.mark.parametrize("dtype", [DataType.fp8_e4m3, DataType.fp8_e5m2], ids=lambda d: d.name)
@pytest.mark.parametrize("options", [{}, {"rotary_dim": 32, "interleaved": True}, {"sequence_axis": 1, "head_dim_axis": 3}], ids=["split", "interleaved_partial", "bshd"])
def test_fp8_storage(stream, options, dtype):
    """8-bit floats are storage only: widened exactly, turned in fp32, rounded once on the way out."""
    rng = np.random.default_rng(39)
    shape = (2, 6, 50, 64)
    x = to_storage(rng.standard_normal(shape).astype(np.float32), dtype)
    plan = run({"y": ex.input("x").rope(**options), "wide": ex.input("x").rope(output_dtype=DataType.fp32, **options)}, {"x": copy_numpy_to_gpu(x, stream, dtype)}, stream)
    assert plan.output("y").get_data_type() == dtype and plan.output("wide").get_data_type() == DataType.fp32
    x32 = from_storage(x, dtype)
    seq = shape[options.get("sequence_axis", 2)]
    want = oracle_rope(x, dtype, options, out_dtype=DataType.fp32).astype(np.float64)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("wide"), stream), want, rtol=0, atol=angle_tolerance(x32, seq, DataType.fp32))
    got = from_storage(copy_gpu_to_numpy(plan.output("y"), stream), dtype).astype(np.float64)
    # one rounding to the 8-bit format: within one unit in the last place of the fp32 result's magnitude
    ulp = np.maximum(2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -9))) - (3 if dtype == DataType.fp8_e4m3 else 2)), 2.0 ** -9)
    assert np.all(np.abs(got - want) <= ulp + 1e-3)


@pytest.mark.parametrize("ids_dtype", [DataType.uint32, DataType.int32, DataType.uint64, DataType.fp32], ids=lambda d: d.name)
def test_position_ids_and_effective_length(stream, ids_dtype):
    rng = np.random.default_rng(32)
    x32 = rng.standard_normal((37, 4, 64)).astype(np.float32)
    positions = rng.integers(0, 500, 37)
    carrier = {DataType.uint32: np.uint32, DataType.int32: np.int32, DataType.uint64: np.uint64, DataType.fp32: np.float32}[ids_dtype]
    inputs = {"x": copy_numpy_to_gpu(x32, stream, DataType.fp32), "p": copy_numpy_to_gpu(positions.astype(carrier), stream, ids_dtype),
              "n": copy_numpy_to_gpu(np.array([300], carrier), stream, ids_dtype)}
    packed = {"sequence_axis": 0, "head_dim_axis": 2}
    ntk = dict(packed, scaling_kind=RotaryScalingKind.dynamic_ntk, scaling_factor=2.0, original_max_position_embeddings=128)
    plan = run({"ids": ex.input("x").rope(position_ids=ex.input("p"), **packed),
                "both": ex.input("x").rope(position_ids=ex.input("p"), effective_sequence_length=ex.input("n"), **ntk),
                "length": ex.input("x").rope(effective_sequence_length=ex.input("n"), **ntk)}, inputs, stream)
    tol = angle_tolerance(x32, 500.0, DataType.fp32)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("ids"), stream), oracle_rope(x32, DataType.fp32, packed, positions), rtol=0, atol=tol)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("both"), stream), oracle_rope(x32, DataType.fp32, ntk, positions, 300), rtol=0, atol=tol)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("length"), stream), oracle_rope(x32, DataType.fp32, ntk, None, 300), rtol=0, atol=tol)
    # the same stamped plan follows the tensors: new positions and a new length, no new kernels
    inputs["p"].copy_from_async(copy_numpy_to_gpu((positions[::-1]).astype(carrier).copy(), stream, ids_dtype), stream)
    inputs["n"].copy_from_async(copy_numpy_to_gpu(np.array([100], carrier), stream, ids_dtype), stream)
    plan.run()
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("both"), stream), oracle_rope(x32, DataType.fp32, ntk, positions[::-1], 100), rtol=0, atol=tol)
    # a short effective length leaves Dynamic NTK unscaled (ExpressionConvenienceOpsTest.cpp:3503-3549 there)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("length"), stream),
                                  copy_gpu_to_numpy(run({"y": ex.input("x").rope(**packed)}, {"x": inputs["x"]}, stream).output("y"), stream))


def test_explicit_positions_equal_the_offset_they_spell_out(stream):
    """ExpressionConvenienceOpsTest.cpp:3627-3668 there, forward and backward."""
    rng = np.random.default_rng(33)
    x32 = rng.standard_normal((1, 2, 9, 16)).astype(np.float32)
    g32 = rng.standard_normal((1, 2, 9, 16)).astype(np.float32)
    tensors = {"x": copy_numpy_to_gpu(x32, stream, DataType.fp32), "positions": copy_numpy_to_gpu(np.arange(9, dtype=np.uint32) + 5, stream, DataType.uint32),
               "__grad_output": copy_numpy_to_gpu(g32, stream, DataType.fp32)}
    with_ids = ex.compile(ex.outputs({"y": ex.input("x").rope(rotary_dim=4, position_ids=ex.input("positions"))}), device_num=0)
    with_offset = ex.compile(ex.outputs({"y": ex.input("x").rope(rotary_dim=4, position_offset=5)}), device_num=0)
    results = []
    for eq, names in ((with_ids, ("x", "positions")), (with_offset, ("x",))):
        plan = eq.stamp({k: tensors[k] for k in names}, stream)
        plan.run()
        back = eq.compile_backward(["x"], error_input_name="__grad_output").stamp({k: tensors[k] for k in names + ("__grad_output",)}, stream)
        back.run()
        results.append((copy_gpu_to_numpy(plan.output("y"), stream), copy_gpu_to_numpy(back.output("x_grad"), stream)))
    np.testing.assert_array_equal(results[0][0], results[1][0])
    np.testing.assert_array_equal(results[0][1], results[1][1])
    with pytest.raises(RuntimeError, match="position_offset == 0"):
        ex.input("x").rope(position_offset=1, position_ids=ex.input("positions"))


BACKWARD = [c for c in CASES if c["name"] in ("plain", "interleaved_partial", "linear", "dynamic_ntk_interleaved", "yarn_explicit_attention_factor_and_betas",
                                               "longrope_long_factors_with_explicit_attention_factor", "llama3_custom_band_and_attention_factor", "bshd",
                                               "packed_position_ids")]


@pytest.mark.parametrize("case", BACKWARD, ids=[c["name"] for c in BACKWARD])
def test_backward_is_the_rotation_turned_back(stream, case):
    """test_rope_compile_backward_preserves_scaling_parameterizations there: x_grad = rope(upstream, inverse)."""
    o = options_of(case)
    shape = case["shape"]
    rng = np.random.default_rng(34)
    x32 = np.array(case["x"], np.float32).reshape(shape)
    g32 = rng.standard_normal(shape).astype(np.float32)
    tensors = {"x": copy_numpy_to_gpu(x32, stream, DataType.fp32), "__grad_output": copy_numpy_to_gpu(g32, stream, DataType.fp32)}
    ids = None
    if case["position_ids"] is not None:
        ids = ex.input("positions")
        tensors["positions"] = copy_numpy_to_gpu(np.array(case["position_ids"], np.uint32), stream, DataType.uint32)
    fwd = ex.compile(ex.outputs({"y": ex.input("x").rope(position_ids=ids, **o)}), device_num=0)
    bwd = fwd.compile_backward(["x"], error_input_name="__grad_output")
    plan = bwd.stamp(tensors, stream)
    plan.run()
    got = copy_gpu_to_numpy(plan.output("x_grad"), stream)
    turned_back = dict(o, inverse=not o.get("inverse", False))
    tol = angle_tolerance(g32, 16.0, DataType.fp32, 1.5)
    np.testing.assert_allclose(got, oracle_rope(g32, DataType.fp32, turned_back, case["position_ids"]), rtol=0, atol=tol)
    # <rope(x), g> = <x, rope^T(g)>
    y = oracle_rope(x32, DataType.fp32, o, case["position_ids"]).astype(np.float64)
    assert abs(float((y * g32).sum()) - float((x32.astype(np.float64) * got).sum())) < 1e-3


def test_walking_and_tiled_kernels_agree(stream, monkeypatch):
    """Layouts with heads between the sequence and the head dimension run the LDS-tiled kernel; switched off, the walking kernel
    takes them: the two work the same angles out and must agree to the last bit.  Different block counts change nothing either."""
    rng = np.random.default_rng(38)
    x = to_storage(rng.standard_normal((3, 130, 5, 64)).astype(np.float32), DataType.bf16)
    t = copy_numpy_to_gpu(x, stream, DataType.bf16)
    options = {"sequence_axis": 1, "head_dim_axis": 3, "rotary_dim": 48, "position_offset": 7}
    results = []
    for env in ({}, {"THOR_ROPE_NO_TILES": "1"}, {"THOR_ROPE_NO_TILES": "1", "THOR_ROPE_BLOCKS": "1"}):
        for name in ("THOR_ROPE_NO_TILES", "THOR_ROPE_BLOCKS"):
            monkeypatch.delenv(name, raising=False)
        for name, value in env.items():
            monkeypatch.setenv(name, value)
        plan = run({"y": ex.input("x").rope(**options)}, {"x": t}, stream)
        results.append((plan.stage_descriptions()[-1], copy_gpu_to_numpy(plan.output("y"), stream)))
    assert "tile=" in results[0][0] and "walk=" in results[1][0] and "walk=15/1," in results[2][0]
    assert np.array_equal(results[0][1], results[1][1]) and np.array_equal(results[1][1], results[2][1])


@pytest.mark.parametrize("dtype", [DataType.bf16, DataType.fp32], ids=lambda d: d.name)
def test_lanes_that_share_pairs_give_the_bits_of_lanes_that_own_them(stream, monkeypatch, dtype):
    """Head dimensions whose halves are not whole 64-byte sectors (80, 96; a partly rotated 128) pair adjacent lanes: each reads,
    turns and writes one of the two vectors of a pair.  Switched off, one lane owns both; the results must be the same bits,
    with a fused elementwise neighbour as well."""
    rng = np.random.default_rng(80)
    for shape, options in (((2, 5, 70, 80), {}), ((1, 3, 129, 96), {"position_offset": 11}), ((2, 2, 64, 128), {"rotary_dim": 80}),
                           ((2, 70, 5, 80), {"sequence_axis": 1, "head_dim_axis": 3}), ((3, 33, 4, 128), {"sequence_axis": 1, "head_dim_axis": 3, "rotary_dim": 48})):
        x = to_storage(rng.standard_normal(shape).astype(np.float32), dtype)
        t = copy_numpy_to_gpu(x, stream, dtype)
        for build in (lambda v: v.rope(**options), lambda v: (v * 2.0 + 1.0).rope(**options) * 0.5):
            results = []
            for off in (False, True):
                monkeypatch.delenv("THOR_ROPE_NO_PAIRED_LANES", raising=False)
                if off:
                    monkeypatch.setenv("THOR_ROPE_NO_PAIRED_LANES", "1")
                plan = run({"y": build(ex.input("x"))}, {"x": t}, stream)
                results.append((plan.stage_descriptions()[-1], copy_gpu_to_numpy(plan.output("y"), stream)))
            half_bytes = options.get("rotary_dim", shape[3]) // 2 * (2 if dtype == DataType.bf16 else 4)
            assert ("paired_lanes" in results[0][0]) == (half_bytes % 64 != 0) and "paired_lanes" not in results[1][0], results[0][0]
            assert np.array_equal(results[0][1], results[1][1])


def test_rotation_inside_a_larger_graph(stream):
    rng = np.random.default_rng(35)
    x32 = rng.standard_normal((2, 3, 40, 32)).astype(np.float32)
    ix = ex.input("x")
    plan = run({"y": (ix * 2.0 + 1.0).rope(rotary_dim=16) * 0.5, "norm": ix.rope().reduce_norm2(axis=3, squeeze=True),
                "of_view": ix.transpose().rope(sequence_axis=3, head_dim_axis=2)}, {"x": copy_numpy_to_gpu(x32, stream, DataType.fp32)}, stream)
    tol = angle_tolerance(2 * x32 + 1, 40.0, DataType.fp32)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("y"), stream),
                               oracle_rope((x32 * np.float32(2) + np.float32(1)), DataType.fp32, {"rotary_dim": 16}) * np.float32(0.5), rtol=0, atol=tol)
    # a rotation keeps the length of every head vector
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("norm"), stream), np.sqrt((x32.astype(np.float64) ** 2).sum(axis=3)), rtol=1e-5)
    swapped = np.ascontiguousarray(np.swapaxes(x32, 2, 3))
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("of_view"), stream),
                               oracle_rope(swapped, DataType.fp32, {"sequence_axis": 3, "head_dim_axis": 2}), rtol=0, atol=tol)


def _neighbour_graphs():
    x, y, z, a = ex.input("x"), ex.input("y"), ex.input("z"), ex.runtime_scalar("a")
    return [
        ("affine_before_scale_after", lambda: (x * 2.0 + 1.0).rope() * 0.5, (2, 3, 40, 32), DataType.fp32, "x"),
        ("products_and_sums_of_three_tensors", lambda: (x * y + z).rope(rotary_dim=16) * y + z * x, (2, 3, 40, 32), DataType.fp32, "xyz"),
        ("transcendental_neighbours", lambda: (x.tanh() * y).rope(interleaved=True).exp() / (z * z + 1.0), (2, 3, 40, 32), DataType.fp32, "xyz"),
        ("runtime_scalar_both_sides", lambda: (x * a + y).rope() * a + 1.0, (2, 3, 40, 32), DataType.fp32, "xya"),
        ("heads_after_sequence", lambda: (x - y).rope(sequence_axis=1, head_dim_axis=3) + z, (2, 40, 3, 32), DataType.fp32, "xyz"),
        ("bf16_every_step_rounded", lambda: (x * y + z).rope() * y - x, (2, 3, 40, 32), DataType.bf16, "xyz"),
        ("fp16_partial_interleaved", lambda: (x + y).rope(rotary_dim=16, interleaved=True) * z, (2, 3, 40, 32), DataType.fp16, "xyz"),
        ("only_after", lambda: x.rope() * y + 0.25, (2, 3, 40, 32), DataType.fp32, "xy"),
        ("only_before", lambda: (x * y).rope(), (2, 3, 40, 32), DataType.fp32, "xy"),
        ("llama3_long_head", lambda: (x * 0.5 + y).rope(scaling_kind=RotaryScalingKind.llama3, scaling_factor=8.0, original_max_position_embeddings=16) - z,
         (1, 2, 64, 128), DataType.bf16, "xyz"),
    ]


@pytest.mark.parametrize("name", [g[0] for g in _neighbour_graphs()])
def test_elementwise_neighbours_run_inside_the_rotation(stream, monkeypatch, name):
    """(x * 2 + 1).rope() * 0.5 is one kernel (one FusedKernel stage there too: RoPE is an operation of the reference's fused kernels)
    and gives, bit for bit, what the plan of separate elementwise and rotation kernels gives."""
    _, build, shape, dtype, used = next(g for g in _neighbour_graphs() if g[0] == name)
    rng = np.random.default_rng(abs(hash(name)) % 1000)
    tensors = {k: copy_numpy_to_gpu(to_storage(rng.standard_normal(shape).astype(np.float32), dtype), stream, dtype) for k in "xyz"}
    results = {}
    for fused in (True, False):
        if fused:
            monkeypatch.delenv("THOR_DISABLE_STAGE_FUSION", raising=False)
        else:
            monkeypatch.setenv("THOR_DISABLE_STAGE_FUSION", "1")
        equation = ex.compile(ex.outputs({"y": build()}), device_num=0)
        plan = equation.stamp({k: t for k, t in tensors.items() if k in used}, stream)
        plan.run({"a": 1.75} if "a" in used else None)
        results[fused] = (plan.stage_kind_names(), plan.stage_descriptions(), copy_gpu_to_numpy(plan.output("y"), stream))
    kinds, descriptions, fused_values = results[True]
    assert kinds == ["FusedKernel"] and descriptions[0].startswith("fused "), descriptions
    assert ("prologue+" in descriptions[0]) == (name != "only_after") and ("+epilogue" in descriptions[0]) == (name != "only_before")
    assert len(results[False][0]) == 1 + (name != "only_after") + (name != "only_before")
    if name == "products_and_sums_of_three_tensors":
        # r * y + z * x: which of the two products joins the addition in one fused multiply-add is the compiler's choice in each
        # kernel; the two results differ by at most the rounding of the product that was rounded on its own
        staged = results[False][2].astype(np.float64)
        zx = np.abs(copy_gpu_to_numpy(tensors["z"], stream).astype(np.float64) * copy_gpu_to_numpy(tensors["x"], stream).astype(np.float64))
        assert np.all(np.abs(fused_values.astype(np.float64) - staged) <= 2.0 ** -23 * (np.abs(staged) + 2 * zx))
    else:
        np.testing.assert_array_equal(fused_values.view(np.uint8), results[False][2].view(np.uint8))


def test_a_rotation_read_twice_or_named_keeps_its_own_tensor(stream):
    rng = np.random.default_rng(39)
    x32 = rng.standard_normal((2, 3, 40, 32)).astype(np.float32)
    ix = ex.input("x")
    turned = (ix * 2.0).rope()
    plan = run({"turned": turned, "half": turned * 0.5, "squared": turned * turned}, {"x": copy_numpy_to_gpu(x32, stream, DataType.fp32)}, stream)
    # the operand is still computed inside the rotation; its two readers share one elementwise kernel
    assert len(plan.stage_kind_names()) == 2 and "prologue+" in plan.stage_descriptions()[0] and "+epilogue" not in plan.stage_descriptions()[0]
    expected = oracle_rope(x32 * np.float32(2), DataType.fp32, {})
    tol = angle_tolerance(2 * x32, 40.0, DataType.fp32)
    got = copy_gpu_to_numpy(plan.output("turned"), stream)
    np.testing.assert_allclose(got, expected, rtol=0, atol=tol)
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("half"), stream), got * np.float32(0.5))
    np.testing.assert_array_equal(copy_gpu_to_numpy(plan.output("squared"), stream), got * got)


def test_output_dtype_and_equal_parameters_share_kernels(stream):
    rng = np.random.default_rng(36)
    x = to_storage(rng.standard_normal((1, 2, 33, 64)).astype(np.float32), DataType.fp16)
    t = copy_numpy_to_gpu(x, stream, DataType.fp16)
    plan = run({"wide": ex.input("x").rope(output_dtype=DataType.fp32, compute_dtype=DataType.fp32), "same": ex.input("x").rope(output_dtype=DataType.fp16)},
               {"x": t}, stream)
    assert plan.output("wide").get_data_type() == DataType.fp32 and plan.output("same").get_data_type() == DataType.fp16
    tol = angle_tolerance(from_storage(x, DataType.fp16), 33.0, DataType.fp32)
    np.testing.assert_allclose(copy_gpu_to_numpy(plan.output("wide"), stream), oracle_rope(x, DataType.fp16, {}, out_dtype=DataType.fp32), rtol=0, atol=tol)
    a, b = ex.input("x").rope(rotary_dim=32, base=500.0), ex.input("x").rope(rotary_dim=32, base=500.0)
    assert a.canonical() == b.canonical() != ex.input("x").rope(rotary_dim=32, base=501.0).canonical()
    shared = run({"a": a, "b": b + 0.0}, {"x": t}, stream)
    assert sum("rope(" in d for d in shared.stage_descriptions()) == 1


def test_validation(stream):
    """test_rope_invalid_rotary_dim_raises_during_expression_construction and test_rope_scaling_parameterization_validation_errors there."""
    q = ex.input("q")
    with pytest.raises(RuntimeError, match="rotary_dim"):
        q.rope(rotary_dim=7)
    bad = [({"scaling_kind": RotaryScalingKind.yarn, "scaling_factor": 2.0}, "original_max_position_embeddings"),
           ({"scaling_kind": RotaryScalingKind.yarn, "scaling_factor": 2.0, "original_max_position_embeddings": 16, "yarn_beta_fast": 0.0}, "beta"),
           ({"scaling_kind": RotaryScalingKind.longrope, "rotary_dim": 8, "scaling_factor": 2.0}, "original_max_position_embeddings"),
           ({"scaling_kind": RotaryScalingKind.longrope, "scaling_factor": 2.0, "original_max_position_embeddings": 16,
             "long_rope_short_factors": [1.0, 1.1, 1.2, 1.3], "long_rope_long_factors": [2.0, 2.2, 2.4, 2.6]}, "explicit rotary_dim"),
           ({"scaling_kind": RotaryScalingKind.longrope, "rotary_dim": 8, "scaling_factor": 2.0, "original_max_position_embeddings": 16,
             "long_rope_short_factors": [1.0, 1.1, 1.2], "long_rope_long_factors": [2.0, 2.2, 2.4, 2.6]}, "rotary_dim / 2"),
           ({"scaling_kind": RotaryScalingKind.longrope, "rotary_dim": 8, "scaling_factor": 2.0, "original_max_position_embeddings": 16,
             "long_rope_short_factors": [1.0, 1.1, 1.2], "long_rope_long_factors": [2.0, 2.2, 2.4]}, "rotary_dim / 2"),
           ({"scaling_kind": RotaryScalingKind.longrope, "rotary_dim": 8, "scaling_factor": 2.0, "original_max_position_embeddings": 16,
             "long_rope_short_factors": [1.0, -1.1, 1.2, 1.3], "long_rope_long_factors": [2.0, 2.2, 2.4, 2.6]}, "short factors"),
           ({"scaling_kind": RotaryScalingKind.llama3, "scaling_factor": 8.0}, "original_max_position_embeddings"),
           ({"scaling_kind": RotaryScalingKind.llama3, "scaling_factor": 8.0, "original_max_position_embeddings": 16, "llama3_low_freq_factor": 4.0,
             "llama3_high_freq_factor": 1.0}, "low_freq_factor < high_freq_factor"),
           ({"base": 0.0}, "base must be positive"), ({"scaling_factor": 0.0}, "scaling factor must be positive"),
           ({"attention_factor": -1.0}, "attention_factor must be positive")]
    for kwargs, match in bad:
        with pytest.raises(RuntimeError, match=match):
            q.rope(output_dtype=DataType.fp16, compute_dtype=DataType.fp32, **kwargs)
    x = copy_numpy_to_gpu(np.zeros((2, 3, 4, 8), np.float32), stream, DataType.fp32)
    with pytest.raises(RuntimeError, match="no larger than the head dimension"):
        run({"y": q.rope(rotary_dim=10)}, {"q": x}, stream)
    with pytest.raises(RuntimeError, match="distinct axes"):
        run({"y": q.rope(sequence_axis=3, head_dim_axis=3)}, {"q": x}, stream)
    with pytest.raises(RuntimeError, match="distinct axes"):
        run({"y": q.rope(sequence_axis=2, head_dim_axis=4)}, {"q": x}, stream)
    with pytest.raises(RuntimeError, match="one position per element of the sequence axis"):
        run({"y": q.rope(position_ids=ex.input("p"))}, {"q": x, "p": copy_numpy_to_gpu(np.zeros(5, np.uint32), stream, DataType.uint32)}, stream)
    with pytest.raises(RuntimeError, match="single element"):
        run({"y": q.rope(effective_sequence_length=ex.input("n"))}, {"q": x, "n": copy_numpy_to_gpu(np.zeros(2, np.uint32), stream, DataType.uint32)}, stream)
    with pytest.raises(RuntimeError, match="floating-point"):
        run({"y": q.rope()}, {"q": copy_numpy_to_gpu(np.zeros((2, 3, 4, 8), np.uint32), stream, DataType.uint32)}, stream)


@pytest.mark.parametrize("dtype", [DataType.bf16, DataType.fp32], ids=lambda d: d.name)
def test_full_size_properties(stream, dtype):
    """[8, 32, 4096, 128]: turning and turning back returns the input (to the storage rounding of two passes), every pair keeps
    its length, and a window of the result matches the oracle."""
    shape = (8, 32, 4096, 128) if dtype == DataType.bf16 else (4, 32, 4096, 128)
    rng = np.random.default_rng(37)
    block = rng.standard_normal((4096, 128)).astype(np.float32)
    x32 = np.broadcast_to(block, shape)
    x = to_storage(np.ascontiguousarray(x32), dtype)
    t = copy_numpy_to_gpu(x, stream, dtype)
    plan = run({"there": ex.input("x").rope(), "back": ex.input("x").rope().rope(inverse=True)}, {"x": t}, stream)
    there = from_storage(copy_gpu_to_numpy(plan.output("there"), stream), dtype)
    back = from_storage(copy_gpu_to_numpy(plan.output("back"), stream), dtype)
    xs = from_storage(x, dtype)
    ulp = {DataType.bf16: 2.0 ** -8, DataType.fp32: 2.0 ** -23}[dtype]  # relative
    # both passes work the same angles out, so their sines and cosines are the same numbers: only roundings remain
    np.testing.assert_allclose(back, xs, rtol=0, atol=3 * ulp * 8 + 1e-5)
    lengths = there[..., :64].astype(np.float64) ** 2 + there[..., 64:].astype(np.float64) ** 2
    np.testing.assert_allclose(lengths, xs[..., :64].astype(np.float64) ** 2 + xs[..., 64:].astype(np.float64) ** 2, rtol=6 * ulp, atol=1e-2 if dtype == DataType.bf16 else 1e-4)
    # every batch and head holds the same plane: the first window against the oracle, every other one against the first
    want = from_storage(oracle_rope(x[:1, :1], dtype, {}), dtype)
    np.testing.assert_allclose(there[:1, :1], want, rtol=0, atol=angle_tolerance(block, 4096.0, dtype))
    assert np.array_equal(there, np.broadcast_to(there[:1, :1], shape))
