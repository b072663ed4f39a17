"""Writes convert_edges.json: fp32 edge-case bit patterns and the fp16 / bf16 / fp8 codes they must convert to.

Expected codes come from witnesses that do not share code with the oracle or the kernels: numpy's float16 cast
(IEEE RNE), the bf16 add-0x7fff identity, and torch's float8 casts for in-range values; NaN -> 0x7fff and fp8
saturate-to-finite (448 / 57344, the reference's KATs in CubReductionDTypeAndLifecycleTest.cpp:205-222) are applied
on top.  Run:  python tests/golden/make_convert_edges.py
"""
import json
import os

import numpy as np
import torch


def f(x):
    return int(np.array([x], dtype=np.float32).view(np.uint32)[0])


bits = [
    0x00000000, 0x80000000, 0x00000001, 0x807FFFFF, 0x00800000,              # zeros, fp32 subnormals, min normal
    f(65504.0), f(65519.99), f(65520.0), f(-65520.0), f(65536.0), f(1e5), f(-1e5),  # fp16 overflow boundary
    f(2.0 ** -24), f(2.0 ** -25), 0x33000001, f(2.0 ** -14), f(2.0 ** -14 * (1 - 2.0 ** -11)), f(6.1e-5), f(5.97e-8), f(2.99e-8),
    0x3F808000, 0x3F818000, 0x3F808001, 0x3F80FFFF, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F7F8000, 0x7F7F7FFF,  # bf16 ties / overflow
    0x7F800000, 0xFF800000, 0x7FC00000, 0xFFC00000, 0x7F800001, 0xFFFFFFFF,   # Inf / NaN
    f(448.0), f(463.9), f(464.0), f(465.0), f(480.0), f(-1000.0), f(2.0 ** -9), f(2.0 ** -10), f(2.0 ** -10 * 1.0001), f(0.0175),
    f(57344.0), f(61439.0), f(61440.0), f(61441.0), f(2.0 ** -16), f(2.0 ** -17), f(2.0 ** -17 * 1.01), f(1.0), f(-1.125), f(0.3),
    f(1.0625), f(1.1875), f(3.0e38), f(1e-40), f(-1e-40),
]
x = np.array(bits, dtype=np.uint32).view(np.float32)
nan = np.isnan(x)

with np.errstate(over="ignore", invalid="ignore"):
    fp16 = x.astype(np.float16).view(np.uint16).copy()
fp16[nan] = 0x7FFF

u = x.view(np.uint32).astype(np.uint64)
bf16 = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
bf16[nan] = 0x7FFF


def fp8(torch_dtype, maxv, maxcode):
    t = torch.from_numpy(np.clip(np.nan_to_num(x, nan=0.0, posinf=maxv, neginf=-maxv), -maxv, maxv))
    codes = t.to(torch_dtype).view(torch.uint8).numpy().copy()
    sign = (x.view(np.uint32) >> 24).astype(np.uint8) & 0x80
    codes[nan] = 0x7F | sign[nan]
    return codes


e4m3 = fp8(torch.float8_e4m3fn, 448.0, 0x7E)
e5m2 = fp8(torch.float8_e5m2, 57344.0, 0x7B)

out = {
    "fp32_bits": [int(b) for b in bits],
    "fp16_bits": [int(v) for v in fp16],
    "bf16_bits": [int(v) for v in bf16],
    "e4m3_bits": [int(v) for v in e4m3],
    "e5m2_bits": [int(v) for v in e5m2],
}
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "convert_edges.json"), "w") as fh:
    json.dump(out, fh, indent=0)
print("wrote", len(bits), "edge vectors")
