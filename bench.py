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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--log2-elements", type=int, default=28)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
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
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "convertSlots<float, f16> (fp32->fp16)", "kernel_avg_ms": round(kernel_avg_ms, 4),
                     "algorithmic_bytes_per_launch": n * BYTES_PER_ELEMENT},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
