"""The five BASELINE configurations at their full sizes, HIP path against the oracle's host restatements of the same workloads
(oracle/thor_oracle_expr.c: expr_config1, rows_f32, softmax_rows_bf16, normalize_rows_f32, relu_scale_bias_f16, channel_stats_f16).

Bars: bit-exact where every operation rounds to a fixed type (fp16 arithmetic, maxima, arg indices); fp32 elementwise results
within the ulp bound that 2-ulp device functions and one fused multiply-add allow; fp32 sums within 1e-5 relative (the order of
the additions differs from the oracle's sequential one)."""
from __future__ import annotations

import numpy as np
import pytest

import oracle
from helpers import copy_gpu_to_numpy, copy_numpy_to_gpu, gpu_tensor, to_storage
from thor_amd import _lib
from thor_amd import physical as ph
from thor_amd.dtypes import DataType
from thor_amd.physical import Expression as ex

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def stream(gpu):
    return ph.Stream(0)


def tiled_on_gpu(block: np.ndarray, copies: int, stream):
    """A device tensor holding `copies` repetitions of a host block (device-to-device copies of one upload)."""
    src = copy_numpy_to_gpu(block, stream, DataType.fp32)
    t = gpu_tensor([block.size * copies], DataType.fp32)
    for k in range(copies):
        _lib.check(_lib.load().thorhip_memcpy_async(t.mem_ptr() + k * block.nbytes, src.mem_ptr(), block.nbytes, 3, stream.handle), "d2d")
    stream.synchronize()
    return t


def test_config1_at_2_to_28_against_the_oracle(stream):
    """out = (a*b + c) * sigmoid(d) over 2^28 fp32 elements: sixteen repetitions of 2^24-element blocks U(-1,1), every element of
    the 1 GiB result compared with oracle.expr_config1 of the block."""
    rng = np.random.default_rng(1234)
    n_block, copies = 1 << 24, 16
    host = {k: rng.uniform(-1, 1, n_block).astype(np.float32) for k in "abcd"}
    tensors = {k: tiled_on_gpu(v, copies, stream) for k, v in host.items()}
    ea, eb, ec, ed = (ex.input(k) for k in "abcd")
    plan = ex.compile((ea * eb + ec) * ed.sigmoid(), 0).stamp(tensors, stream)
    assert plan.stage_kind_names() == ["FusedKernel"] and "flat(vec=4)" in plan.stage_descriptions()[0]
    plan.run()
    got = copy_gpu_to_numpy(plan.output(), stream).reshape(copies, n_block)
    want, _ = oracle.expr_config1(host["a"], host["b"], host["c"], host["d"])
    # the oracle rounds a*b and the sum separately, the kernel may fuse them (the reference compiles with -fmad=true): one ulp of
    # the larger term of the cancelling sum, carried through the product with sigmoid(d) <= 1; plus 2-ulp exp twice, the division
    # and the final product: 4 ulp of the result
    a64, b64, c64 = (host[k].astype(np.float64) for k in "abc")
    bound = (4 * np.spacing(np.abs(want)) + np.spacing(np.maximum(np.abs(a64 * b64), np.abs(c64)).astype(np.float32))).astype(np.float64)
    for k in range(copies):
        assert np.all(np.abs(got[k].astype(np.float64) - want.astype(np.float64)) <= bound), f"repetition {k}"
    np.testing.assert_array_equal(got[0], got[copies - 1])  # equal inputs, equal results wherever they lie in the tensor


def test_config3_against_the_oracle(stream):
    """fp32 [8192, 8192] N(0,1): row sums, row maxima, row argmax and the full sum against oracle.rows_f32."""
    rng = np.random.default_rng(1236)
    x = rng.standard_normal((8192, 8192), dtype=np.float32)
    t = copy_numpy_to_gpu(x, stream, DataType.fp32)
    rows = ph.CubReduction(ph.CubReductionOp.Sum, 1, DataType.fp32).stamp(t, stream)
    rmax = ph.CubReduction(ph.CubReductionOp.Max, 1, DataType.fp32).stamp(t, stream)
    amax = ph.CubArgReduction(ph.CubArgReductionOp.ArgMax, 1, produce_value=False).stamp(t, stream)
    full = ph.CubReduction(ph.CubReductionOp.Sum, [0, 1], DataType.fp32).stamp(t, stream)
    for s in (rows, rmax, amax, full):
        s.run()
    want_sum, want_max, want_arg, _ = oracle.rows_f32(x)
    got_sum = copy_gpu_to_numpy(rows.get_output_tensor(), stream).reshape(-1)
    np.testing.assert_array_equal(copy_gpu_to_numpy(rmax.get_output_tensor(), stream).reshape(-1), want_max)
    got_arg = copy_gpu_to_numpy(amax.get_index_output_tensor(), stream).reshape(-1)
    assert got_arg.dtype == np.uint32
    np.testing.assert_array_equal(got_arg, want_arg)
    # sums of 8192 N(0,1) values: |sum| ~ 90 while the summed magnitude is ~6500, so a different order of the fp32 additions moves
    # the result by up to ~1e-7 * 6500.  The bound is 1e-5 relative to the result wherever the result is not small (|sum| above a
    # hundredth of the summed magnitude) and 1e-5 of that hundredth elsewhere (cancellation).
    magnitude = np.abs(x).astype(np.float64).sum(axis=1)
    exact = x.astype(np.float64).sum(axis=1)
    scale = np.maximum(np.abs(exact), 1e-2 * magnitude)
    assert np.all(np.abs(got_sum - exact) <= 1e-5 * scale)
    assert np.all(np.abs(want_sum - exact) <= 1e-5 * scale)  # the oracle's sequential sum meets the same bound
    large = np.abs(exact) >= 1e-2 * magnitude
    assert large.sum() > 1000
    np.testing.assert_allclose(got_sum[large], want_sum[large], rtol=2e-5)
    got_full = float(copy_gpu_to_numpy(full.get_output_tensor(), stream).reshape(-1)[0])
    assert abs(got_full - exact.sum()) <= 1e-5 * max(abs(exact.sum()), 1e-3 * magnitude.sum())


def test_config4_softmax_full_size_against_the_oracle(stream):
    """y = exp(x - rowmax) / rowsum over bf16 [16384, 4096], x ~ N(0,3), fp32 arithmetic and output: every row against
    oracle.softmax_rows_bf16 at 1e-5 relative."""
    rng = np.random.default_rng(1237)
    shape = (16384, 4096)
    x = to_storage(rng.standard_normal(shape, dtype=np.float32) * 3, DataType.bf16)
    ix = ex.input("x")
    e = (ix - ix.reduce_max(axis=1)).exp()
    plan = ex.compile(e / e.reduce_sum(axis=1), 0).stamp({"x": copy_numpy_to_gpu(x, stream, DataType.bf16)}, stream)
    assert plan.stage_kind_names() == ["FusedRowKernel"]
    plan.run()
    got = copy_gpu_to_numpy(plan.output(), stream)
    assert got.dtype == np.float32 and got.shape == shape
    want, _ = oracle.softmax_rows_bf16(x)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-37)
    np.testing.assert_allclose(got.sum(axis=1, dtype=np.float64), 1.0, rtol=1e-5)


def test_config4_normalize_full_size_against_the_oracle(stream):
    """(x - mean) / sqrt(var + 1e-5) over fp32 [32768, 1024], population variance: every row against oracle.normalize_rows_f32."""
    rng = np.random.default_rng(1237)
    y = rng.standard_normal((32768, 1024), dtype=np.float32) * 4 + 1
    iy = ex.input("y")
    centered = iy - iy.reduce_mean(axis=1)
    expr = centered / ((centered * centered).reduce_mean(axis=1) + 1e-5).sqrt()
    plan = ex.compile(expr, 0).stamp({"y": copy_numpy_to_gpu(y, stream, DataType.fp32)}, stream)
    assert plan.stage_kind_names() == ["FusedRowKernel"]
    plan.run()
    got = copy_gpu_to_numpy(plan.output(), stream)
    want, _ = oracle.normalize_rows_f32(y, 1e-5)
    # centred values cancel (|x - mean| can be far below |x|): an error of the fp32 mean of ~1e-7 * |mean| shifts every element
    # by that much, so the bound has an absolute part of 1e-5 of the row's scale (the normalised values are O(1))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    z = got.astype(np.float64)
    np.testing.assert_allclose(z.mean(axis=1), 0.0, atol=2e-6)
    np.testing.assert_allclose((z * z).mean(axis=1), 1.0, rtol=2e-5)


def test_config5_full_size_against_the_oracle(stream):
    """fp16 NCHW [64, 256, 56, 56]: y = relu(x * scale + bias) bit for bit against oracle.relu_scale_bias_f16, per-channel sum and
    sum of squares against oracle.channel_stats_f16; as separate plans and as the one-pass plan with three outputs."""
    rng = np.random.default_rng(1238)
    shape = (64, 256, 56, 56)
    x = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)
    scale = rng.uniform(0.5, 1.5, (1, 256, 1, 1)).astype(np.float32).astype(np.float16)
    bias = rng.uniform(-0.1, 0.1, (1, 256, 1, 1)).astype(np.float32).astype(np.float16)
    want_y, _ = oracle.relu_scale_bias_f16(x, scale.reshape(-1), bias.reshape(-1))
    want_sum, want_sq, _ = oracle.channel_stats_f16(x)
    x64 = x.astype(np.float64)
    exact_sum = x64.sum(axis=(0, 2, 3))
    sq16 = (x * x).astype(np.float64)  # numpy rounds the fp16 product to fp16, like a materialised fp16 stage
    exact_sq = sq16.sum(axis=(0, 2, 3))
    magnitude = np.abs(x64).sum(axis=(0, 2, 3))
    del x64, sq16
    tx = copy_numpy_to_gpu(x, stream, DataType.fp16)
    ts = copy_numpy_to_gpu(scale, stream, DataType.fp16)
    tb = copy_numpy_to_gpu(bias, stream, DataType.fp16)
    ix = ex.input("x")
    y = (ix * ex.input("scale") + ex.input("bias")).max(0.0)
    stats = {"sum": ix.reduce_sum(axis=[0, 2, 3], squeeze=True), "sumsq": (ix * ix).reduce_sum(axis=[0, 2, 3], squeeze=True)}

    def check_stats(outs, label):
        got_sum = copy_gpu_to_numpy(outs("sum"), stream).reshape(-1).astype(np.float64)
        got_sq = copy_gpu_to_numpy(outs("sumsq"), stream).reshape(-1).astype(np.float64)
        assert np.all(np.abs(got_sum - exact_sum) <= 1e-5 * np.maximum(np.abs(exact_sum), 1e-2 * magnitude)), label
        np.testing.assert_allclose(got_sq, exact_sq, rtol=1e-5, err_msg=label)
        # the oracle adds 200 704 values per channel one after the other in fp32: its own error is ~1e-4 relative, so it bounds
        # the GPU result only that loosely; the float64 sums above are the tight check
        np.testing.assert_allclose(got_sq, want_sq, rtol=1e-3, err_msg=label)
        assert np.all(np.abs(got_sum - want_sum) <= 1e-3 * magnitude), label

    relu = ex.compile(y, 0).stamp({"x": tx, "scale": ts, "bias": tb}, stream)
    assert relu.stage_kind_names() == ["FusedKernel"] and "broadcast(" in relu.stage_descriptions()[0]
    relu.run()
    np.testing.assert_array_equal(copy_gpu_to_numpy(relu.output(), stream).view(np.uint16), want_y.view(np.uint16))
    del relu
    two = ex.compile(ex.outputs(stats), 0).stamp({"x": tx}, stream)
    assert two.stage_kind_names() == ["FusedReduction"]
    two.run()
    check_stats(two.output, "sum and sum of squares in one pass")
    del two
    three = ex.compile(ex.outputs({"y": y, **stats}), 0).stamp({"x": tx, "scale": ts, "bias": tb}, stream)
    assert three.stage_kind_names() == ["FusedReduction"], three.stage_descriptions()
    three.run()
    np.testing.assert_array_equal(copy_gpu_to_numpy(three.output("y"), stream).view(np.uint16), want_y.view(np.uint16))
    check_stats(three.output, "relu and both statistics in one pass")
    single = ph.CubReduction(ph.CubReductionOp.Sum, [0, 2, 3], DataType.fp32).stamp(tx, stream)
    single.run()
    got = copy_gpu_to_numpy(single.get_output_tensor(), stream).reshape(-1).astype(np.float64)
    assert np.all(np.abs(got - exact_sum) <= 1e-5 * np.maximum(np.abs(exact_sum), 1e-2 * magnitude))
