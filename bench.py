"""Headline benchmark: BASELINE config 2, the TypeConverter round trip on 2^28 elements, on one MI355X.

One step = fp32->fp16, fp16->fp32, fp32->bf16, bf16->fp32 over 2^28 elements resident in HBM (6 algorithmic bytes per
element per conversion).  Prints ONE JSON line: whole-step HBM GB/s, the roofline of the dominant kernel (fp32->fp16)
timed with HIP events on the launch stream, and the CPU oracle's rate on a bounded sample as the CPU baseline.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E published peak
# HBM bytes one fp32->fp16 launch over 2^28 elements moves, from rocprofv3 FETCH_SIZE + WRITE_SIZE runs scaled by the
# same counters' readings for a plain copy kernel of known size (profiles/convert_round_trip_2p28_hbm_traffic.txt).
MEASURED_TRAFFIC_BYTES_2P28 = 1_610_591_764  # 1023.98 MiB fetched + 512.00 MiB written
BYTES_PER_ELEMENT = 6   # fp32 <-> 16-bit: 4 + 2


def c2_block(n, seed=1235):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(n).astype(np.float32)
    x[0::100] *= np.float32(1e5)
    x[1::100] *= np.float32(1e-40)
    return x


def cpu_baseline(seconds_budget: float = 12.0):
    """Times the CPU oracle (a port of TypeConverter::cpuConvertTypeImpl, same thread-partition rule) on a bounded
    sample of the same workload: the four conversions over 2^25-element windows until the budget is used."""
    import oracle
    oracle.build()
    n = 1 << 25
    x = c2_block(n)
    h = np.empty(n, dtype=np.float16)
    b = np.empty(n, dtype=np.uint16)
    w = np.empty(n, dtype=np.float32)
    threads = 1
    elems = 0
    t0 = time.perf_counter()
    while True:
        threads = oracle.convert_raw(x.ctypes.data, h.ctypes.data, oracle.FP32, oracle.FP16, n)
        oracle.convert_raw(h.ctypes.data, w.ctypes.data, oracle.FP16, oracle.FP32, n)
        oracle.convert_raw(x.ctypes.data, b.ctypes.data, oracle.FP32, oracle.BF16, n)
        oracle.convert_raw(b.ctypes.data, w.ctypes.data, oracle.BF16, oracle.FP32, n)
        elems += 4 * n
        dt = time.perf_counter() - t0
        if dt >= seconds_budget:
            break
    gbps = elems * BYTES_PER_ELEMENT / dt / 1e9
    return {"value": round(gbps, 3), "unit": "GB/s", "cores": int(threads), "kind": "port",
            "sample": f"{elems // (4 * n)} passes of the 4 conversions over 2^25 elements ({dt:.1f} s)"}


def cpu_baseline_other_configs(seconds_each: float = 1.5):
    """The oracle's host restatements of configs 1, 3, 4, 5 (OpenMP over all host cores) on bounded samples of the same
    workloads; GB/s on the same algorithmic bytes as the GPU lines."""
    import oracle
    oracle.build()
    rng = np.random.default_rng(99)
    out = {}

    def timed(name, fn, nbytes, sample):
        threads = fn()  # warm-up, also pages the buffers in
        reps, t0 = 0, time.perf_counter()
        while True:
            threads = fn()
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= seconds_each:
                break
        out[name] = {"GB/s": round(nbytes * reps / dt / 1e9, 2), "cores": int(threads), "kind": "port", "sample": f"{reps} passes over {sample} ({dt:.1f} s)"}

    n = 1 << 24
    a, b, c, d = (rng.uniform(-1, 1, n).astype(np.float32) for _ in range(4))
    timed("c1_fused_elementwise_fp32", lambda: oracle.expr_config1(a, b, c, d)[1], 20 * n, "2^24 elements")
    del a, b, c, d
    x = rng.standard_normal((2048, 8192), dtype=np.float32)
    timed("c3_row_sum_max_argmax_fp32", lambda: oracle.rows_f32(x)[3], 4 * x.size, "[2048, 8192] (sum, max and argmax in one pass)")
    xs = oracle.convert((rng.standard_normal((2048, 4096), dtype=np.float32) * 3), oracle.FP32, oracle.BF16)
    timed("c4_softmax_bf16", lambda: oracle.softmax_rows_bf16(xs)[1], 6 * xs.size, "[2048, 4096]")
    xn = rng.standard_normal((8192, 1024), dtype=np.float32)
    timed("c4_normalize_fp32", lambda: oracle.normalize_rows_f32(xn)[1], 8 * xn.size, "[8192, 1024]")
    xc = rng.standard_normal((8, 256, 56, 56), dtype=np.float32).astype(np.float16)
    sc = rng.uniform(0.5, 1.5, 256).astype(np.float16)
    bi = rng.uniform(-0.1, 0.1, 256).astype(np.float16)
    timed("c5_relu_scale_bias_fp16", lambda: oracle.relu_scale_bias_f16(xc, sc, bi)[1], 4 * xc.size, "[8, 256, 56, 56]")
    timed("c5_channel_sum_and_sumsq_fp16", lambda: oracle.channel_stats_f16(xc)[2], 2 * xc.size, "[8, 256, 56, 56]")
    return out


def bench_other_configs(only=None):
    """BASELINE configs 1, 3, 4, 5 through the Expression / reduction API: GB/s on algorithmic bytes, HIP-event timed.  `only`: substrings;
    a line whose name holds none of them is set up but not launched (for short profiler runs)."""
    from thor_amd import physical as ph
    from thor_amd.dtypes import DataType
    from thor_amd.physical import Expression as ex
    from thor_amd.runtime import Event

    stream = ph.Stream(0)
    results = {}

    class RawStream:  # Event.record wants an object with .handle
        handle = stream.handle

    def gpu_from(values, dtype):
        """fp32 host values -> a device tensor of `dtype`: the copy converts on the GPU (Tensor::copyFromAsync), so the GPU legs of the
        bench need nothing but the product library."""
        values = np.ascontiguousarray(values, dtype=np.float32)
        shape = list(values.shape)
        cpu = ph.PhysicalTensor(ph.Placement(ph.DeviceType.cpu), ph.PhysicalTensor.Descriptor(DataType.fp32, shape))
        cpu.numpy()[...] = values
        gpu = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(dtype, shape))
        gpu.copy_from_async(cpu, stream)
        stream.synchronize()
        return gpu

    def clone(t):
        c = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(t.get_data_type(), t.get_dimensions()))
        c.copy_from_async(t, stream)
        stream.synchronize()
        return c

    def timed(name, runs, nbytes, elements, note=""):
        """Median of 5 samples; a sample is one pass over every rotating buffer (at least 8 launches), bracketed by events on
        the launch stream (the reference's protocol: warm-up, >= 5 samples x >= 4 iterations, median)."""
        if only and not any(part in name for part in only):
            return
        if callable(runs):
            runs = [runs]
        reps = max(8, len(runs))
        for k in range(max(3, len(runs))):
            runs[k % len(runs)]()
        stream.synchronize()
        samples = []
        for _ in range(5):
            a, b = Event(), Event()
            a.record(RawStream)
            for k in range(reps):
                runs[k % len(runs)]()
            b.record(RawStream)
            b.synchronize()
            samples.append(a.elapsed_ms(b) / reps)
        ms = float(np.median(samples))
        results[name] = {"ms": round(ms, 4), "GB/s": round(nbytes / ms / 1e6, 1), "pct_hbm_peak": round(100 * nbytes / ms / 1e6 / HBM_PEAK_GBPS, 1),
                         "Gelem/s": round(elements / ms / 1e6, 2), "rotating_buffers": len(runs), "plan": note}

    rng = np.random.default_rng(1234)
    # ---- config 1: out = (a*b+c)*sigmoid(d), fp32, 2^20 (cache resident by construction) and 2^28 (5 GiB per launch)
    for log2n in (20, 28):
        n = 1 << log2n
        block = rng.uniform(-1, 1, min(n, 1 << 22)).astype(np.float32)
        tensors = {}
        for k in "abcd":
            t = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp32, [n]))
            src = gpu_from(np.roll(block, ord(k)), DataType.fp32)
            from thor_amd import _lib
            for off in range(0, n, block.size):
                _lib.check(_lib.load().thorhip_memcpy_async(t.mem_ptr() + off * 4, src.mem_ptr(), block.nbytes, 3, stream.handle), "d2d")
            stream.synchronize()
            tensors[k] = t
        ea, eb, ec, ed = (ex.input(k) for k in "abcd")
        plan = ex.compile((ea * eb + ec) * ed.sigmoid(), 0).stamp(tensors, stream)
        timed(f"c1_fused_elementwise_fp32_2^{log2n}", plan.run, 20 * n, n, "+".join(plan.stage_descriptions()))
        del tensors, plan

    # ---- config 3: fp32 [8192, 8192] (256 MiB per input; rotated over 6 copies)
    x = gpu_from(rng.standard_normal((8192, 8192), dtype=np.float32), DataType.fp32)
    n = 8192 * 8192
    xs3 = [x] + [clone(x) for _ in range(5)]
    for name, op, axes in (("c3_full_sum", ph.CubReductionOp.Sum, [0, 1]), ("c3_row_sum", ph.CubReductionOp.Sum, 1),
                           ("c3_row_max", ph.CubReductionOp.Max, 1), ("c3_col_sum", ph.CubReductionOp.Sum, 0)):
        stamps = [ph.CubReduction(op, axes, DataType.fp32).stamp(t, stream) for t in xs3]
        timed(name, [st.run for st in stamps], 4 * n, n, stamps[0].get_kernel_variant())
    amax = [ph.CubArgReduction(ph.CubArgReductionOp.ArgMax, 1, produce_value=False).stamp(t, stream) for t in xs3]
    timed("c3_row_argmax", [a.run for a in amax], 4 * n, n, amax[0].get_kernel_variant())
    del x, xs3, stamps, amax

    # ---- config 4: bf16 [16384, 4096] softmax (fp32 out), fp32 [32768, 1024] mean/variance normalise
    xs = gpu_from((rng.standard_normal((16384, 4096), dtype=np.float32) * 3), DataType.bf16)
    ix = ex.input("x")
    e = (ix - ix.reduce_max(axis=1)).exp()
    soft = ex.compile(e / e.reduce_sum(axis=1), 0)
    n = 16384 * 4096
    xs4 = [xs] + [clone(xs) for _ in range(3)]
    for label, env in (("staged", "1"), ("fused", "0")):
        os.environ["THOR_DISABLE_ROW_FUSION"] = env
        plans = [soft.stamp({"x": t}, stream) for t in xs4]
        timed(f"c4_softmax_bf16_{label}", [p_.run for p_ in plans], 6 * n, n, ">".join(plans[0].stage_kind_names()) + " " + plans[0].stage_descriptions()[0])
        del plans
    del xs, xs4
    xn = gpu_from(rng.standard_normal((32768, 1024), dtype=np.float32), DataType.fp32)
    mean = ix.reduce_mean(axis=1)
    cen = ix - mean
    var = (cen * cen).reduce_mean(axis=1)
    norm = ex.compile(cen / (var + 1e-5).sqrt(), 0)
    n = 32768 * 1024
    xn4 = [xn] + [clone(xn) for _ in range(5)]
    for label, env in (("staged", "1"), ("fused", "0")):
        os.environ["THOR_DISABLE_ROW_FUSION"] = env
        plans = [norm.stamp({"x": t}, stream) for t in xn4]
        timed(f"c4_normalize_fp32_{label}", [p_.run for p_ in plans], 8 * n, n, ">".join(plans[0].stage_kind_names()) + " " + plans[0].stage_descriptions()[0])
        del plans
    os.environ.pop("THOR_DISABLE_ROW_FUSION", None)
    del xn, xn4

    # ---- config 5: fp16 NCHW [64,256,56,56] (98 MiB per tensor; rotated over 8 copies)
    shape = (64, 256, 56, 56)
    xc = gpu_from(rng.standard_normal(shape, dtype=np.float32), DataType.fp16)
    scale = gpu_from(rng.uniform(0.5, 1.5, (1, 256, 1, 1)).astype(np.float32), DataType.fp16)
    bias = gpu_from(rng.uniform(-0.1, 0.1, (1, 256, 1, 1)).astype(np.float32), DataType.fp16)
    n = int(np.prod(shape))
    xc8 = [xc] + [clone(xc) for _ in range(7)]
    relu = ex.compile((ex.input("x") * ex.input("scale") + ex.input("bias")).max(0.0), 0)
    plans = [relu.stamp({"x": t, "scale": scale, "bias": bias}, stream) for t in xc8]
    timed("c5_relu_scale_bias_fp16", [p_.run for p_ in plans], 4 * n, n, "+".join(plans[0].stage_descriptions()))
    csum = [ph.CubReduction(ph.CubReductionOp.Sum, [0, 2, 3], DataType.fp32).stamp(t, stream) for t in xc8]
    timed("c5_channel_sum_fp16", [c.run for c in csum], 2 * n, n, csum[0].get_kernel_variant())
    stats = ex.compile(ex.outputs({"sum": ix.reduce_sum(axis=[0, 2, 3], squeeze=True), "sumsq": (ix * ix).reduce_sum(axis=[0, 2, 3], squeeze=True)}), 0)
    plans = [stats.stamp({"x": t}, stream) for t in xc8]
    timed("c5_channel_sum_and_sumsq_fp16", [p_.run for p_ in plans], 2 * n, n, ">".join(plans[0].stage_kind_names()) + " " + plans[0].stage_descriptions()[0])
    y = (ex.input("x") * ex.input("scale") + ex.input("bias")).max(0.0)
    all3 = ex.compile(ex.outputs({"y": y, "sum": ix.reduce_sum(axis=[0, 2, 3], squeeze=True), "sumsq": (ix * ix).reduce_sum(axis=[0, 2, 3], squeeze=True)}), 0)
    plans = [all3.stamp({"x": t, "scale": scale, "bias": bias}, stream) for t in xc8]
    timed("c5_relu_and_channel_statistics_one_pass_fp16", [p_.run for p_ in plans], 4 * n, n,
          ">".join(plans[0].stage_kind_names()) + " " + plans[0].stage_descriptions()[0])
    del xc, xc8, plans, csum
    # the same kernels on four times the batch ([256, 256, 56, 56], 392 MiB per tensor): a launch on the BASELINE tensor lasts 18 us, so its
    # ramp and tail weigh on its rate; these lines show what the kernels stream at once they run long enough
    shape4 = (256, 256, 56, 56)
    n4 = int(np.prod(shape4))
    big = [ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp16, list(shape4))) for _ in range(3)]
    quarter = gpu_from(rng.standard_normal(shape, dtype=np.float32), DataType.fp16)
    for t in big:
        for part in range(4):
            _lib.check(_lib.load().thorhip_memcpy_async(t.mem_ptr() + part * n * 2, quarter.mem_ptr(), n * 2, 3, stream.handle), "d2d")
    stream.synchronize()
    csum = [ph.CubReduction(ph.CubReductionOp.Sum, [0, 2, 3], DataType.fp32).stamp(t, stream) for t in big]
    timed("c5_channel_sum_fp16_batch256", [c.run for c in csum], 2 * n4, n4, csum[0].get_kernel_variant())
    plans = [stats.stamp({"x": t}, stream) for t in big]
    timed("c5_channel_sum_and_sumsq_fp16_batch256", [p_.run for p_ in plans], 2 * n4, n4, ">".join(plans[0].stage_kind_names()) + " " + plans[0].stage_descriptions()[0])
    plans = [relu.stamp({"x": t, "scale": scale, "bias": bias}, stream) for t in big[:2]]
    timed("c5_relu_scale_bias_fp16_batch256", [p_.run for p_ in plans], 4 * n4, n4, "+".join(plans[0].stage_descriptions()))
    del big, quarter, plans, csum

    # ---- ragged batches (the rows next to the dense path): [2^22, 64] fp32 values (1 GiB) in 65 536 segments of log-normal
    # length; bytes counted are the values read once (reductions), written once (broadcast), read + written once (softmax)
    rows, width, segments = 1 << 22, 64, 1 << 16
    weights = rng.lognormal(0.0, 1.0, segments)
    cuts = np.floor(np.cumsum(weights) / weights.sum() * rows).astype(np.int64)
    host_offsets = ph.PhysicalTensor(ph.Placement(ph.DeviceType.cpu), ph.PhysicalTensor.Descriptor(DataType.uint32, [segments + 1]))
    host_offsets.numpy()[...] = np.concatenate([[0], cuts[:-1], [rows]]).astype(np.uint32)
    offsets_u32 = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.uint32, [segments + 1]))
    offsets_u32.copy_from_async(host_offsets, stream)
    stream.synchronize()
    from thor_amd import _lib
    block = gpu_from(rng.standard_normal((1 << 16, width), dtype=np.float32), DataType.fp32)
    values = []
    for _ in range(3):
        t = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp32, [rows, width]))
        for off in range(0, rows * width, (1 << 16) * width):
            _lib.check(_lib.load().thorhip_memcpy_async(t.mem_ptr() + off * 4, block.mem_ptr(), (1 << 16) * width * 4, 3, stream.handle), "d2d")
        values.append(t)
    stream.synchronize()
    n = rows * width
    sums = [ph.CubSegmentedReduction(ph.CubReductionOp.Sum, DataType.fp32).stamp_runtime_offsets(
        t, ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp32, [segments, width])), offsets_u32, stream)
        for t in values]
    timed("ragged_segment_sum_fp32", [s_.run for s_ in sums], 4 * n, n, sums[0].get_kernel_variant())
    args = [ph.CubSegmentedArgReduction(ph.CubArgReductionOp.ArgMax).stamp_runtime_offsets(
        t, ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.uint64, [segments, width])), offsets_u32, stream)
        for t in values]
    timed("ragged_segment_argmax_fp32", [a_.run for a_ in args], 4 * n, n, args[0].get_kernel_variant())
    per_segment = sums[0].get_output_tensor()
    rv, ro = ex.input("x.values"), ex.input("x.offsets")
    # stamped once like every other line (the one-call form, ph.segmented_broadcast, builds its kernel's text on every call: about
    # 280 us of host time per call, more than the launch takes)
    spread_plan = ex.compile(ex.outputs({"rows": ex.input("per_segment").segmented_broadcast(ro, segments, rows, width)}), 0)
    plans = [spread_plan.stamp({"per_segment": per_segment, "x.offsets": offsets_u32}, stream, preallocated_outputs={"rows": t}) for t in values]
    timed("ragged_segmented_broadcast_fp32", [p_.run for p_ in plans], 4 * n, n, " | ".join(plans[0].stage_descriptions()))
    del plans, spread_plan
    spread = lambda v: v.segmented_broadcast(ro, segments, rows, width)
    shifted = rv - spread(rv.segment_max(ro, segments, rows, width))
    soft = (shifted.exp() / spread(shifted.exp().segment_sum(ro, segments, rows, width))).with_ragged_runtime_extent(ro, segments, rows, width)
    ragged = ex.compile(ex.outputs({"y": soft}), 0)
    for label, env in (("staged", "1"), ("fused", "0")):
        os.environ["THOR_DISABLE_STAGE_FUSION"] = env
        plans = [ragged.stamp({"x.values": t, "x.offsets": offsets_u32}, stream) for t in values[:2]]
        timed(f"ragged_segment_softmax_fp32_{label}", [p_.run for p_ in plans], 8 * n, n,
              ">".join(plans[0].stage_kind_names()) + " " + " | ".join(plans[0].stage_descriptions()))
        del plans
    os.environ.pop("THOR_DISABLE_STAGE_FUSION", None)
    del values, sums, args, per_segment, block

    # ---- backward equations (compile_backward): bytes counted are every operand and the upstream gradient read once and every
    # gradient written once
    n = 1 << 26
    fill = gpu_from(rng.uniform(0.5, 1.5, 1 << 22).astype(np.float32), DataType.fp32)
    tensors = {}
    for k in ("a", "b", "c", "d", "__grad_output"):
        t = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp32, [n]))
        for off in range(0, n, 1 << 22):
            _lib.check(_lib.load().thorhip_memcpy_async(t.mem_ptr() + off * 4, fill.mem_ptr(), 4 << 22, 3, stream.handle), "d2d")
        tensors[k] = t
    stream.synchronize()
    ea, eb, ec, ed = (ex.input(k) for k in "abcd")
    plan = ex.compile((ea * eb + ec) * ed.sigmoid(), 0).compile_backward(["a", "b", "c", "d"], error_input_name="__grad_output").stamp(tensors, stream)
    timed("backward_c1_four_gradients_fp32_2^26", plan.run, 36 * n, n, ">".join(plan.stage_kind_names()) + " " + plan.stage_descriptions()[0])
    del tensors, plan, fill
    xs = gpu_from((rng.standard_normal((16384, 4096), dtype=np.float32) * 3), DataType.bf16)
    gs = gpu_from(rng.standard_normal((16384, 4096), dtype=np.float32), DataType.bf16)
    n = 16384 * 4096
    pairs = [(xs, gs), (clone(xs), clone(gs)), (clone(xs), clone(gs))]
    soft_backward = ex.compile(ex.input("x").softmax(), 0).compile_backward(["x"], error_input_name="__grad_output")
    plans = [soft_backward.stamp({"x": a_, "__grad_output": g_}, stream) for a_, g_ in pairs]
    timed("backward_c4_softmax_bf16", [p_.run for p_ in plans], 6 * n, n, ">".join(plans[0].stage_kind_names()) + " " + plans[0].stage_descriptions()[0])
    del xs, gs, pairs, plans
    x = gpu_from(rng.standard_normal((8192, 8192), dtype=np.float32), DataType.fp32)
    n = 8192 * 8192
    row_max_backward = ex.compile(ex.input("x").reduce_max(axis=1, squeeze=[1]), 0).compile_backward(["x"])
    plans = [row_max_backward.stamp({"x": t}, stream) for t in (x, clone(x), clone(x))]
    timed("backward_c3_row_max_fp32", [p_.run for p_ in plans], 8 * n, n, ">".join(plans[0].stage_kind_names()) + " " + " | ".join(plans[0].stage_descriptions()))
    del plans

    # ---- prefix scans (Expression.scan): bytes counted are the values read once and the result written once
    from thor_amd.physical import ScanOp
    xs3 = [x, clone(x), clone(x)]
    row_sum = ex.compile(ex.input("x").scan(ScanOp.sum), 0)
    plans = [row_sum.stamp({"x": t}, stream) for t in xs3]
    timed("scan_c3_row_cumsum_fp32", [p_.run for p_ in plans], 8 * n, n, plans[0].stage_descriptions()[0])
    row_argmax = ex.compile(ex.input("x").scan(ScanOp.arg_max), 0)
    plans = [row_argmax.stamp({"x": t}, stream) for t in xs3]
    timed("scan_c3_row_running_argmax_fp32", [p_.run for p_ in plans], 8 * n, n, plans[0].stage_descriptions()[0])
    # gradient of the running maximum: reads x and the upstream gradient, writes the gradient (12 B/element)
    gs3 = [clone(x), clone(x), clone(x)]
    row_max_scan_backward = ex.compile(ex.input("x").scan(ScanOp.max), 0).compile_backward(["x"], error_input_name="__grad_output")
    plans = [row_max_scan_backward.stamp({"x": t, "__grad_output": g_}, stream) for t, g_ in zip(xs3, gs3)]
    timed("backward_scan_c3_row_running_max_fp32", [p_.run for p_ in plans], 12 * n, n, " | ".join(plans[0].stage_descriptions()))
    del gs3
    flat = ex.compile(ex.input("x").reshape([n]).scan(ScanOp.sum), 0)
    plans = [flat.stamp({"x": t}, stream) for t in xs3]
    timed("scan_flat_cumsum_fp32_2^26", [p_.run for p_ in plans], 8 * n, n, plans[0].stage_descriptions()[0])
    del plans, xs3, x
    xb = gpu_from(rng.standard_normal((16384, 4096), dtype=np.float32), DataType.bf16)
    nb = 16384 * 4096
    xb3 = [xb, clone(xb), clone(xb)]
    plans = [row_sum.stamp({"x": t}, stream) for t in xb3]
    timed("scan_c4_row_cumsum_bf16", [p_.run for p_ in plans], 4 * nb, nb, plans[0].stage_descriptions()[0])
    del plans, xb3, xb
    scalars = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp32, [rows * 16]))
    wide_offsets = ph.PhysicalTensor(ph.Placement(ph.DeviceType.cpu), ph.PhysicalTensor.Descriptor(DataType.uint32, [segments + 1]))
    wide_offsets.numpy()[...] = host_offsets.numpy() * 16
    ragged_offsets = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.uint32, [segments + 1]))
    ragged_offsets.copy_from_async(wide_offsets, stream)
    stream.synchronize()
    ragged_sum = ex.compile(ex.input("v").segmented_scan(ex.input("o"), ScanOp.sum), 0)
    plan = ragged_sum.stamp({"v": scalars, "o": ragged_offsets}, stream)
    timed("scan_ragged_cumsum_fp32_2^26", plan.run, 8 * rows * 16, rows * 16, plan.stage_descriptions()[0])
    del plan, scalars

    # ---- rotary position embedding (Expression.rope): every element read once and written once
    from thor_amd.dtypes import size_of
    from thor_amd.physical import RotaryScalingKind
    plane = rng.standard_normal((4096, 128), dtype=np.float32)
    for label, dtype, shape, options in (
            ("rope_bf16_bhsd_8x32x4096x128", DataType.bf16, (8, 32, 4096, 128), {}),
            ("rope_bf16_bshd_llama3_8x4096x32x128", DataType.bf16, (8, 4096, 32, 128),
             {"sequence_axis": 1, "head_dim_axis": 3, "scaling_kind": RotaryScalingKind.llama3, "scaling_factor": 8.0, "original_max_position_embeddings": 8192,
              "base": 500000.0}),
            ("rope_fp32_bhsd_interleaved_4x32x4096x128", DataType.fp32, (4, 32, 4096, 128), {"interleaved": True})):
        q = gpu_from(np.resize(plane, shape), dtype)
        count = int(np.prod(shape))
        rope = ex.compile(ex.input("q").rope(**options), 0)
        plans = [rope.stamp({"q": t}, stream) for t in (q, clone(q))]
        timed(label, [p_.run for p_ in plans], 2 * size_of(dtype) * count, count, plans[0].stage_descriptions()[0])
        del plans, q

    # ---- select-flagged and top-k (the selection primitives next to the scans): bytes counted are the keys / values and flags read
    # once and the selected elements written once
    n = 1 << 26
    keys = gpu_from(np.resize(rng.standard_normal(1 << 22).astype(np.float32), n), DataType.fp32)
    flag_block = (rng.random(1 << 22) < 0.5).astype(np.uint8)
    flags = gpu_from(np.resize(flag_block, n), DataType.uint8)
    kept = int(np.resize(flag_block, n).sum())
    selected = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp32, [n]))
    count = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.uint32, [1]))
    plan = ph.SelectionPlan.select_flagged(keys, flags, selected, count)
    temp = plan.allocate_temp_storage()
    timed("select_flagged_fp32_2^26_half_kept", lambda: plan.run(temp, keys, flags, selected, count, stream=stream), 5 * n + 4 * kept, n, plan.variant())
    del flags, selected, plan, temp
    for k in (64, 65536):
        best = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp32, [k]))
        plan = ph.SelectionPlan.top_k(keys, best, k)
        temp = plan.allocate_temp_storage()
        timed(f"topk_fp32_2^26_k{k}", lambda: plan.run(temp, keys, best, stream=stream), 4 * n + 4 * k, n, plan.variant())
        del plan, temp, best
    del keys
    rows_k = gpu_from(np.resize(rng.standard_normal(1 << 22).astype(np.float32), (16384, 4096)), DataType.bf16)
    best = ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.bf16, [16384, 64]))
    plan = ph.SelectionPlan.top_k(rows_k, best, 64, segment_size=4096, num_segments=16384)
    temp = plan.allocate_temp_storage()
    timed("topk_rows_bf16_16384x4096_k64", lambda: plan.run(temp, rows_k, best, stream=stream), 2 * 16384 * 4096 + 2 * 16384 * 64, 16384 * 4096,
          plan.variant())
    del rows_k, best, plan, temp

    # ---- a reduction whose output's fastest axis is not the input's: fp32 storage [512, 8, 16384] seen as [16384, 8, 512], summed over
    # the middle axis into a dense [16384, 512] (written through an LDS transpose)
    storage = [ph.PhysicalTensor(ph.Placement(ph.DeviceType.gpu, 0), ph.PhysicalTensor.Descriptor(DataType.fp32, [512, 8, 16384])) for _ in range(3)]
    for t in storage:
        t.memset_async(0, stream)
    stream.synchronize()
    views = [t.alias_view([16384, 8, 512], [1, 16384, 8 * 16384]) for t in storage]
    permuted = [ph.CubReduction(ph.CubReductionOp.Sum, [1], DataType.fp32).stamp(v, stream) for v in views]
    timed("permuted_output_sum_fp32_16384x8x512_view", [p_.run for p_ in permuted], 4 * 512 * 8 * 16384 + 4 * 512 * 16384, 512 * 8 * 16384,
          permuted[0].get_kernel_variant())
    del storage, views, permuted
    return results


def _short(name, width=70):
    import re
    name = re.sub(r"\(anonymous namespace\)::", "", name)
    name = re.sub(r"^void ", "", name)
    return name if len(name) <= width else name[:width]


def _bench_lines_by_kernel_tag(bench_json):
    """kernel-name tag (the 8 hex digits every generated kernel carries) -> the bench lines whose plan names it."""
    import re
    if not bench_json:
        return {}
    record = json.loads(open(bench_json).read().strip().splitlines()[-1])
    tags = {}
    for line, v in record.get("other_configs", {}).items():
        for tag in re.findall(r"\[[a-z_]+_([0-9a-f]{8})\]", v.get("plan", "")):
            tags.setdefault(tag, []).append(line)
    return tags


def _line_of(kernel_name, tags):
    for tag, lines in tags.items():
        if tag in kernel_name:
            return ",".join(sorted(set(lines)))
    return ""


def summarize_kernel_trace(db, bench_json=None):
    """Per-kernel dispatch durations out of the rocpd database a `rocprofv3 --kernel-trace --stats` run of this script wrote."""
    import sqlite3
    con = sqlite3.connect(db)
    tags = _bench_lines_by_kernel_tag(bench_json)
    rows = list(con.execute("select name, count(*), avg(end-start), min(end-start), max(end-start), sum(end-start) from kernels group by name order by 6 desc"))
    total = sum(r[5] for r in rows) or 1
    print(f"{'calls':>6} {'avg_us':>10} {'min_us':>10} {'max_us':>10} {'total_ms':>10} {'pct':>6}  {'kernel':70s} bench line")
    for name, calls, avg, lo, hi, tot in rows:
        print(f"{calls:6d} {avg/1e3:10.2f} {lo/1e3:10.2f} {hi/1e3:10.2f} {tot/1e6:10.3f} {100*tot/total:6.2f}  {_short(name):70s} {_line_of(name, tags)}")


def summarize_hbm_traffic(fetch_db, write_db, bench_json=None):
    """HBM bytes per dispatch out of two `rocprofv3 --pmc` runs (FETCH_SIZE, then WRITE_SIZE) of this script with --calibration-copy:
    each counter is scaled by its own reading for the calibration copy (uint32 -> int32 over 2^28 elements: 1 GiB each way).  Dispatches
    of one kernel with different grids (the same conversion kernel also prepares smaller inputs) are listed apart."""
    import sqlite3
    tags = _bench_lines_by_kernel_tag(bench_json)

    def read(db, counter):
        con = sqlite3.connect(db)
        return {(n, g): (c, a) for n, g, c, a in con.execute(
            "select kernel_name, grid_size, count(*), avg(value) from counters_collection where counter_name=? group by kernel_name, grid_size", (counter,))}
    fetch, write = read(fetch_db, "FETCH_SIZE"), read(write_db, "WRITE_SIZE")
    calibration = max((key for key in fetch if "convertSlots<unsigned int, int" in key[0]), key=lambda key: key[1])
    kf, kw = 1048576.0 / fetch[calibration][1], 1048576.0 / write[calibration][1]
    print(f"calibration copy {_short(calibration[0], 48)}: FETCH_SIZE {fetch[calibration][1]:.1f} KiB, WRITE_SIZE {write[calibration][1]:.1f} KiB "
          f"per dispatch for 1 048 576 KiB each way -> factors {kf:.5f}, {kw:.5f}")
    print(f"{'dispatches':>10} {'grid':>11} {'fetch MiB':>10} {'write MiB':>10} {'total MB':>10}  kernel <- bench line")
    for key in sorted(fetch, key=lambda k: -(fetch[k][1] * kf + write.get(k, (0, 0))[1] * kw)):
        fm, wm = fetch[key][1] * kf / 1024, write.get(key, (0, 0))[1] * kw / 1024
        print(f"{fetch[key][0]:10d} {key[1]:11d} {fm:10.2f} {wm:10.2f} {(fm + wm) * 1.048576:10.2f}  {_short(key[0])} <- {_line_of(key[0], tags)}")


def summarize_counters(dbs, bench_json=None):
    """Average per dispatch of every counter in one or more `rocprofv3 --pmc` databases of this script: one row per kernel and grid
    size, one column per counter, plus the average dispatch duration of the first database that saw the kernel."""
    import sqlite3
    tags = _bench_lines_by_kernel_tag(bench_json)
    table, names = {}, []
    for db in dbs:
        con = sqlite3.connect(db)
        for kernel, grid, counter, count, avg, duration in con.execute(
                "select kernel_name, grid_size, counter_name, count(*), avg(value), avg(duration) from counters_collection "
                "group by kernel_name, grid_size, counter_name"):
            row = table.setdefault((kernel, grid), {"dispatches": count, "us": duration / 1e3})
            row[counter] = avg
            if counter not in names:
                names.append(counter)
    for at in range(0, len(names), 4):
        group = names[at:at + 4]
        print(f"{'dispatches':>10} {'grid':>11} {'avg_us':>9} " + " ".join(f"{n:>36s}" for n in group) + "  kernel <- bench line")
        for (kernel, grid), row in sorted(table.items(), key=lambda item: -item[1]["us"]):
            if not any(n in row for n in group) or row["us"] < 15.0:
                continue
            print(f"{row['dispatches']:10d} {grid:11d} {row['us']:9.1f} " + " ".join(f"{row.get(n, float('nan')):36.1f}" for n in group) +
                  f"  {_short(kernel, 44)} <- {_line_of(kernel, tags)}")
        print()
    # Ratios that say where a memory-bound kernel waits.  The *_sum counters add up the L2 channel instances (16 per XCD, 8 XCDs),
    # so a ratio of two of them is per instance; a level counter divided by its request counter is the mean time a request was
    # outstanding (Little's law), in L2 clocks.
    instances = 128.0
    derived = [
        ("L2 busy %", lambda r: 100 * r["TCC_BUSY_sum"] / r["TCC_CYCLE_sum"]),
        ("L2 miss %", lambda r: 100 * r["TCC_MISS_sum"] / (r["TCC_HIT_sum"] + r["TCC_MISS_sum"])),
        ("rd req", lambda r: r["TCC_EA0_RDREQ_sum"]),
        ("wr req", lambda r: r["TCC_EA0_WRREQ_sum"]),
        ("rd latency clk", lambda r: r["TCC_EA0_RDREQ_LEVEL_sum"] / r["TCC_EA0_RDREQ_sum"]),
        ("rd in flight", lambda r: r["TCC_EA0_RDREQ_LEVEL_sum"] / (r["TCC_CYCLE_sum"] / instances)),
        ("L2 MHz", lambda r: r["TCC_CYCLE_sum"] / instances / r["us"]),
        ("rd credit stall %", lambda r: 100 * r["TCC_EA0_RDREQ_DRAM_CREDIT_STALL_sum"] / r["TCC_CYCLE_sum"]),
        ("wr credit stall %", lambda r: 100 * r["TCC_EA0_WRREQ_DRAM_CREDIT_STALL_sum"] / r["TCC_CYCLE_sum"]),
        ("wr req stall %", lambda r: 100 * r["TCC_EA0_WRREQ_STALL_sum"] / r["TCC_CYCLE_sum"]),
        ("tag stall %", lambda r: 100 * r["TCC_TAG_STALL_sum"] / r["TCC_CYCLE_sum"]),
        ("wave wait %", lambda r: 100 * r["SQ_WAIT_INST_ANY"] / r["SQ_WAVE_CYCLES"]),
    ]
    usable = []
    for title, ratio in derived:
        try:
            ratio(max(table.values(), key=lambda r: r["us"]))
            usable.append((title, ratio))
        except (KeyError, ZeroDivisionError):
            pass
    if usable:
        print("derived per dispatch (sums over the 128 L2 channel instances; latency and in-flight counts by Little's law):")
        print(f"{'grid':>11} {'avg_us':>9} " + " ".join(f"{title:>17s}" for title, _ in usable) + "  kernel <- bench line")
        for (kernel, grid), row in sorted(table.items(), key=lambda item: -item[1]["us"]):
            if row["us"] < 15.0:
                continue
            cells = []
            for _, ratio in usable:
                try:
                    cells.append(f"{ratio(row):17.1f}")
                except (KeyError, ZeroDivisionError):
                    cells.append(f"{'-':>17s}")
            print(f"{grid:11d} {row['us']:9.1f} " + " ".join(cells) + f"  {_short(kernel, 44)} <- {_line_of(kernel, tags)}")



def run_experiment(name):
    """A/B experiments whose tables are kept under profiles/ (each prints plain text; medians of 7 samples of 4 launches, HIP events on
    the launch stream).  c1_address_stagger: config 1 at 2^28 with the four operands and the output shifted inside their allocations,
    so that a wavefront's four loads do not start on the same offset of their 4 KiB pages ("c1_address_stagger:BYTES": that step only).  c1_tensor_spacing: the five tensors
    inside one allocation, 1 GiB plus a given distance apart ("c1_tensor_spacing:0,4,8": those MiB counts).  c1_operand_streams: the same size with 1,
    2, 3 and 4 operands read per element written, a plain sum against config 1's arithmetic.  c1_sigmoid_exponentials: config 1 with
    the stable sigmoid's two exponentials as written against the shared one.  c4_row_kernel_shapes: the two row kernels of config 4 with
    other lane counts per row than the planner's and with several rows per block taken in turn.  stage_overlap: plans with independent branches on
    helper streams (THOR_STAGE_OVERLAP=1) against one lane."""
    from thor_amd import physical as ph
    from thor_amd.dtypes import DataType
    from thor_amd.physical import Expression as ex
    from thor_amd.runtime import Event

    name, _, only = name.partition(":")  # "c1_address_stagger:4352" runs the one line with steps of that many bytes (for counter runs)
    stream = ph.Stream(0)

    class RawStream:
        handle = stream.handle

    gpu = ph.Placement(ph.DeviceType.gpu, 0)

    def time_runs(runs, launches=4, samples=7):
        for run in runs:
            run()
        stream.synchronize()
        taken = []
        for _ in range(samples):
            first, last = Event(), Event()
            first.record(RawStream)
            for k in range(launches):
                runs[k % len(runs)]()
            last.record(RawStream)
            last.synchronize()
            taken.append(first.elapsed_ms(last) / launches)
        return float(np.median(taken))

    def device_tensor(values, dtype=DataType.fp32):
        values = np.ascontiguousarray(values, dtype=np.float32)
        host = ph.PhysicalTensor(ph.Placement(ph.DeviceType.cpu), ph.PhysicalTensor.Descriptor(DataType.fp32, list(values.shape)))
        host.numpy()[...] = values
        device = ph.PhysicalTensor(gpu, ph.PhysicalTensor.Descriptor(dtype, list(values.shape)))
        device.copy_from_async(host, stream)
        stream.synchronize()
        return device

    n = 1 << 28
    if name in ("c1_address_stagger", "c1_operand_streams", "c1_sigmoid_exponentials"):
        room = 1 << 22  # 16 MiB of slack per tensor
        base = {k: ph.PhysicalTensor(gpu, ph.PhysicalTensor.Descriptor(DataType.fp32, [n + room])) for k in "abcdo"}
        # the bench line's data (uniform in [-1, 1), a 2^22 block repeated): tensors of zeros stream 5-6 % faster
        from thor_amd import _lib
        block = np.random.default_rng(1234).uniform(-1, 1, 1 << 22).astype(np.float32)
        for k, t in base.items():
            source = device_tensor(np.roll(block, ord(k)))
            for off in range(0, n + room, block.size):
                _lib.check(_lib.load().thorhip_memcpy_async(t.mem_ptr() + off * 4, source.mem_ptr(), block.nbytes, 3, stream.handle), "d2d")
            stream.synchronize()
        a, b, c, d = (ex.input(k) for k in "abcd")
        c1 = (a * b + c) * d.sigmoid()

        def line(label, expression, offsets, reads):
            equation = ex.compile(ex.outputs({"o": expression}), 0)
            names = "abcd"[:reads]
            views = {k: base[k].alias_view([n], [1], element_offset=offsets[i]) for i, k in enumerate(names)}
            out = base["o"].alias_view([n], [1], element_offset=offsets[4])
            plan = equation.stamp(views, stream, preallocated_outputs={"o": out})
            ms = time_runs([plan.run])
            moved = 4 * (reads + 1) * n
            print(f"{label:44s} {ms * 1000:8.1f} us  {moved / ms / 1e6:7.0f} GB/s  {moved / ms / 1e6 / 8000:.3f}  {plan.stage_descriptions()[0][:50]}", flush=True)

        if name == "c1_address_stagger":
            print("operand base addresses:", {k: hex(t.mem_ptr()) for k, t in base.items()}, flush=True)
            page = 1024  # elements per 4 KiB
            for label, step in (("no stagger", 0), ("256 B steps", 64), ("1 KiB steps", 256), ("4 KiB steps", page), ("16 KiB steps", 4 * page),
                                ("64 KiB steps", 16 * page), ("256 KiB steps", 64 * page), ("1 MiB steps", 256 * page), ("4 KiB + 256 B steps", page + 64),
                                ("no stagger (again)", 0)):
                if not only or int(only) == step * 4:
                    line(label, c1, [i * step for i in range(5)], 4)
        elif name == "c1_operand_streams":
            for round_ in range(2):
                line(f"round {round_}: a*2 (1 read : 1 write)", a * 2.0, [0] * 5, 1)
                line(f"round {round_}: a+b (2 : 1)", a + b, [0] * 5, 2)
                line(f"round {round_}: a+b+c (3 : 1)", a + b + c, [0] * 5, 3)
                line(f"round {round_}: a+b+c+d (4 : 1)", a + b + c + d, [0] * 5, 4)
                line(f"round {round_}: (a*b+c)*sigmoid(d) (4 : 1)", c1, [0] * 5, 4)
        else:
            for round_ in range(3):
                os.environ["THOR_SIGMOID_TWO_EXPONENTIALS"] = "1"
                line(f"round {round_}: two exponentials", c1, [0] * 5, 4)
                os.environ.pop("THOR_SIGMOID_TWO_EXPONENTIALS")
                line(f"round {round_}: shared exponential", c1, [0] * 5, 4)
        return
    if name == "c1_tensor_spacing":
        # the five tensors of config 1 inside one allocation, a fixed distance apart: what the distance between the streams does
        a, b, c, d = (ex.input(k) for k in "abcd")
        equation = ex.compile(ex.outputs({"o": (a * b + c) * d.sigmoid()}), 0)
        room = 1 << 24
        pool = ph.PhysicalTensor(gpu, ph.PhysicalTensor.Descriptor(DataType.fp32, [5 * (n + room)]))
        from thor_amd import _lib
        block = device_tensor(np.random.default_rng(1234).uniform(-1, 1, 1 << 22).astype(np.float32))
        for off in range(0, 5 * (n + room), 1 << 22):
            _lib.check(_lib.load().thorhip_memcpy_async(pool.mem_ptr() + off * 4, block.mem_ptr(), 4 << 22, 3, stream.handle), "d2d")
        stream.synchronize()
        print("pool at", hex(pool.mem_ptr()), flush=True)
        spacings = (0, 128, 256, 1024, 4096, 65536, 1 << 20, 2 << 20, 4 << 20, 20 << 20, (20 << 20) + 4096, 33 << 20, 48 << 20, 0)
        if only:
            spacings = tuple(int(v) << 20 for v in only.split(","))  # "c1_tensor_spacing:0,1,2,3": those MiB counts
        for extra_bytes in spacings:
            stride = n + extra_bytes // 4
            views = {k: pool.alias_view([n], [1], element_offset=i * stride) for i, k in enumerate("abcd")}
            out = pool.alias_view([n], [1], element_offset=4 * stride)
            plan = equation.stamp(views, stream, preallocated_outputs={"o": out})
            ms = time_runs([plan.run])
            print(f"tensors 1 GiB + {extra_bytes:>9d} B apart   {ms * 1000:8.1f} us  {20 * n / ms / 1e6 / 8000:.3f}", flush=True)
        return
    if name == "c4_row_kernel_shapes":
        rng = np.random.default_rng(0)
        ix = ex.input("x")
        e = (ix - ix.reduce_max(axis=1)).exp()
        centred = ix - ix.reduce_mean(axis=1)
        lines = (("softmax bf16 -> fp32 [16384, 4096]", ex.compile(e / e.reduce_sum(axis=1), 0), (16384, 4096), DataType.bf16, 6, (64, 128, 256, 512)),
                 ("normalise fp32 [32768, 1024]", ex.compile(centred / ((centred * centred).reduce_mean(axis=1) + 1e-5).sqrt(), 0), (32768, 1024), DataType.fp32, 8,
                  (32, 64, 128, 256)))
        for label, equation, shape, dtype, bytes_per_element, lane_counts in lines:
            first = device_tensor(rng.standard_normal(shape, dtype=np.float32) * 3, dtype)
            copies = [first]
            for _ in range(3):
                copy = ph.PhysicalTensor(gpu, ph.PhysicalTensor.Descriptor(dtype, list(shape)))
                copy.copy_from_async(first, stream)
                copies.append(copy)
            stream.synchronize()
            moved = bytes_per_element * shape[0] * shape[1]

            def measure(what, switches):
                for key, value in switches.items():
                    os.environ[key] = str(value)
                plans = [equation.stamp({"x": t}, stream) for t in copies]
                for key in switches:
                    os.environ.pop(key)
                ms = time_runs([p.run for p in plans], launches=8)
                print(f"{label:36s} {what:28s} {ms * 1000:7.1f} us  {moved / ms / 1e6 / 8000:.3f}  {plans[0].stage_descriptions()[0][:90]}", flush=True)

            measure("the planner's choice", {})
            for lanes in lane_counts:
                measure(f"{lanes} lanes per row", {"THOR_ROW_THREADS": lanes})
            for turns in (2, 4, 8):
                measure(f"{turns} rows per block in turn", {"THOR_ROW_TURNS": turns})
            del copies, first
        return
    if name == "stage_overlap":
        def clone(t):
            c = ph.PhysicalTensor(gpu, ph.PhysicalTensor.Descriptor(t.get_data_type(), t.get_dimensions()))
            c.copy_from_async(t, stream)
            stream.synchronize()
            return c

        def compare(label, plans):
            taken = {"forked": [], "one lane": []}
            for _ in range(7):
                os.environ["THOR_STAGE_OVERLAP"] = "1"
                taken["forked"].append(time_runs([p.run for p in plans], launches=24, samples=1))
                os.environ["THOR_STAGE_OVERLAP"] = "0"
                taken["one lane"].append(time_runs([p.run for p in plans], launches=24, samples=1))
            print(f"{label:44s} forked {np.median(taken['forked']) * 1e3:8.1f} us   one lane {np.median(taken['one lane']) * 1e3:8.1f} us   "
                  f"stages {plans[0].stage_kind_names()}", flush=True)

        rng = np.random.default_rng(0)
        x = device_tensor(rng.standard_normal((8192, 8192), dtype=np.float32))
        backward = ex.compile(ex.input("x").reduce_max(axis=1, squeeze=[1]), 0).compile_backward(["x"])
        compare("backward of row max, 8192^2", [backward.stamp({"x": t}, stream) for t in (x, clone(x), clone(x))])
        y = device_tensor(rng.standard_normal((4096, 8192), dtype=np.float32))
        two = ex.compile(ex.input("x").reduce_sum(axis=1).reduce_sum(axis=[0, 1]) + ex.input("y").reduce_max(axis=1).reduce_sum(axis=[0, 1]), 0)
        compare("two large independent reductions", [two.stamp({"x": x, "y": y}, stream)])
        small = [device_tensor(rng.standard_normal((64, 256 + 8 * k), dtype=np.float32)) for k in range(4)]
        total = None
        for k in range(4):
            term = ex.input(f"s{k}").reduce_sum(axis=1).reduce_sum(axis=[0, 1])
            total = term if total is None else total + term
        chains = ex.compile(total, 0)
        compare("four small independent reduction chains", [chains.stamp({f"s{k}": t for k, t in enumerate(small)}, stream)])
        return
    raise SystemExit(f"unknown experiment {name!r}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--summarize-kernel-trace", nargs="+", metavar=("DB", "BENCH_JSON"),
                    help="print the per-kernel duration table of a rocprofv3 --kernel-trace database (optionally tagged with the bench lines of BENCH_JSON) and exit")
    ap.add_argument("--summarize-hbm-traffic", nargs="+", metavar=("FETCH_DB", "WRITE_DB"),
                    help="print the HBM-traffic table of two rocprofv3 --pmc databases (FETCH_SIZE run, WRITE_SIZE run[, BENCH_JSON]) and exit")
    ap.add_argument("--summarize-counters", nargs="+", metavar="DB",
                    help="print the average reading per dispatch of every counter in the given rocprofv3 --pmc databases, kernel by kernel "
                         "(a last argument ending in .json is taken as BENCH_JSON), and exit")
    ap.add_argument("--lines", default="", help="comma-separated substrings: launch only the secondary lines whose name holds one of them")
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--log2-elements", type=int, default=28)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the secondary lines for BASELINE configs 1, 3, 4, 5")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="before the timed region, launch a plain copy kernel of known size (uint32->int32 over the same element count: "
                         "4 B read + 4 B written per element) so that hardware counters of a profiled run can be scaled against it")
    ap.add_argument("--experiment", default="", metavar="NAME",
                    help="run one A/B experiment instead of the bench and print its table: c1_address_stagger, c1_operand_streams, "
                         "c1_tensor_spacing, c1_sigmoid_exponentials, c4_row_kernel_shapes or stage_overlap")
    args = ap.parse_args()
    if args.experiment:
        run_experiment(args.experiment)
        return
    if args.summarize_kernel_trace:
        summarize_kernel_trace(*args.summarize_kernel_trace[:2])
        return
    if args.summarize_hbm_traffic:
        summarize_hbm_traffic(*args.summarize_hbm_traffic[:3])
        return
    if args.summarize_counters:
        given = list(args.summarize_counters)
        bench_json = given.pop() if given[-1].endswith(".json") else None
        summarize_counters(given, bench_json)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    from thor_amd import runtime
    from thor_amd.dtypes import DataType
    from thor_amd.runtime import DeviceBuffer, Event, Stream, TypeConverter

    assert runtime.device_count() >= 1, "bench.py needs a GPU"
    runtime.set_device(0)
    info = runtime.device_info(0)
    stream = Stream(0)
    n = 1 << args.log2_elements

    block = c2_block(min(n, 1 << 24))
    src = DeviceBuffer(n * 4)
    for k in range(n // block.size):
        src.upload(np.roll(block, k * 9973), stream, offset_bytes=k * block.nbytes)
    f16, b16 = DeviceBuffer(n * 2), DeviceBuffer(n * 2)
    w16, wb16 = DeviceBuffer(n * 4), DeviceBuffer(n * 4)

    def step(events=None):
        if events is not None:
            events[0].record(stream)
        TypeConverter.convert_type(src.ptr, f16.ptr, DataType.fp32, DataType.fp16, n, stream)
        if events is not None:
            events[1].record(stream)
        TypeConverter.convert_type(f16.ptr, w16.ptr, DataType.fp16, DataType.fp32, n, stream)
        TypeConverter.convert_type(src.ptr, b16.ptr, DataType.fp32, DataType.bf16, n, stream)
        TypeConverter.convert_type(b16.ptr, wb16.ptr, DataType.bf16, DataType.fp32, n, stream)

    if args.calibration_copy:
        for _ in range(3):
            TypeConverter.convert_type(src.ptr, w16.ptr, DataType.uint32, DataType.int32, n, stream)
        stream.synchronize()
    for _ in range(args.warmup):
        step()
    stream.synchronize()
    runtime.device_synchronize()

    pairs = [(Event(), Event()) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for k in range(args.steps):
        step(pairs[k])
    stream.synchronize()
    runtime.device_synchronize()
    elapsed = time.perf_counter() - t0

    step_bytes = 4 * n * BYTES_PER_ELEMENT
    value = step_bytes * args.steps / elapsed / 1e9
    kernel_ms = [a.elapsed_ms(b) for a, b in pairs]
    kernel_avg_ms = float(np.mean(kernel_ms))
    achieved = n * BYTES_PER_ELEMENT / (kernel_avg_ms * 1e-3) / 1e9

    result = {
        "metric": "fused-expression/reduction/convert HBM GB/s and % of MI355X peak BW; Gelem/s",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"TypeConverter round trip fp32->fp16->fp32 and fp32->bf16->fp32 on 2^{args.log2_elements} elements "
                               "(N(0,1), 1% x1e5, 1% x1e-40); 4 conversions x 6 B/element per step",
                   "elements": n, "device": info.name.decode(), "arch": info.arch_name.decode(), "compute_units": info.compute_units},
        "gelem_per_s": round(4 * n * args.steps / elapsed / 1e9, 3),
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES_2P28 if args.log2_elements == 28 else None,
                     "kernel": "convertSlots<float, thor::f16, 4, 1> (fp32->fp16)", "kernel_avg_ms": round(kernel_avg_ms, 4),
                     "algorithmic_bytes_per_launch": n * BYTES_PER_ELEMENT},
    }
    for b_ in (src, f16, b16, w16, wb16):
        b_.free()
    if not args.no_other_configs:
        result["other_configs"] = bench_other_configs([part for part in args.lines.split(",") if part] or None)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
        if not args.no_other_configs:
            result["cpu_baseline_other_configs"] = cpu_baseline_other_configs()
    if not args.no_other_configs:
        # The fraction of the HBM peak of every line, as the last key of the JSON line so that it survives in a record that keeps
        # only the end of the output: the BASELINE configurations first (C2's four directions together, then C1, C3, C4, C5 in
        # the order bench_other_configs runs them), the lines next to the path after them.
        fractions = {"c2_convert_round_trip_2^%d" % args.log2_elements: round(value / HBM_PEAK_GBPS, 4),
                     "c2_convert_fp32_to_fp16": round(achieved / HBM_PEAK_GBPS, 4)}
        fractions.update({name: round(v["GB/s"] / HBM_PEAK_GBPS, 4) for name, v in result["other_configs"].items()})
        result["per_config_frac"] = fractions
    print(json.dumps(result))


if __name__ == "__main__":
    main()
