"""Pins the CPU oracle's converters (oracle/thor_oracle.c) against independent witnesses: the x86 F16C hardware
converter over all 2^32 fp32 bit patterns, the add-0x7fff bf16 formulation, numpy float16, torch CPU bfloat16 /
float8 casts, and the reference's own fp8 saturation KATs
(test/Utilities/TensorOperations/CubReductionDTypeAndLifecycleTest.cpp:205-222 -> 448 / 57344)."""
import json
import os

import numpy as np
import pytest

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_fp16_narrowing_exhaustive_against_f16c():
    bad = oracle.lib().oracle_check_f16_against_f16c()
    if bad < 0:
        pytest.skip("host CPU has no F16C")
    assert bad == 0


def test_fp16_widening_all_codes_against_f16c():
    bad = oracle.lib().oracle_check_f16_widen_against_f16c()
    if bad < 0:
        pytest.skip("host CPU has no F16C")
    assert bad == 0


def test_bf16_narrowing_exhaustive_against_add_trick():
    assert oracle.lib().oracle_check_bf16_against_addtrick() == 0


def _c2_like(n, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(n).astype(np.float32)
    x[0::100] *= np.float32(1e5)
    x[1::100] *= np.float32(1e-40)
    return x


def test_fp16_matches_numpy_on_config_shaped_data():
    x = _c2_like(1 << 20, 1235)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = oracle.convert(x, oracle.FP32, oracle.FP16).view(np.uint16)
    assert np.array_equal(got, want)
    back = oracle.convert(got.view(np.float16), oracle.FP16, oracle.FP32)
    assert np.array_equal(back.view(np.uint32), want.view(np.float16).astype(np.float32).view(np.uint32))


def test_bf16_matches_torch_on_config_shaped_data():
    torch = pytest.importorskip("torch")
    x = _c2_like(1 << 20, 1235)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.convert(x, oracle.FP32, oracle.BF16)
    assert np.array_equal(got, want)
    back = oracle.convert(got, oracle.BF16, oracle.FP32)
    assert np.array_equal(back.view(np.uint32), want.astype(np.uint32) << 16)


def test_golden_edge_vectors():
    with open(os.path.join(GOLDEN, "convert_edges.json")) as f:
        g = json.load(f)
    x = np.array(g["fp32_bits"], dtype=np.uint32).view(np.float32)
    assert np.array_equal(oracle.convert(x, oracle.FP32, oracle.FP16).view(np.uint16), np.array(g["fp16_bits"], dtype=np.uint16))
    assert np.array_equal(oracle.convert(x, oracle.FP32, oracle.BF16), np.array(g["bf16_bits"], dtype=np.uint16))
    assert np.array_equal(oracle.convert(x, oracle.FP32, oracle.FP8_E4M3), np.array(g["e4m3_bits"], dtype=np.uint8))
    assert np.array_equal(oracle.convert(x, oracle.FP32, oracle.FP8_E5M2), np.array(g["e5m2_bits"], dtype=np.uint8))


@pytest.mark.parametrize("dt,torch_name,maxv", [(oracle.FP8_E4M3, "float8_e4m3fn", 448.0), (oracle.FP8_E5M2, "float8_e5m2", 57344.0)])
def test_fp8_codes_and_saturation(dt, torch_name, maxv):
    torch = pytest.importorskip("torch")
    tdt = getattr(torch, torch_name)
    codes = np.arange(256, dtype=np.uint8)
    f = oracle.convert(codes, dt, oracle.FP32)
    tf = torch.from_numpy(codes).view(tdt).to(torch.float32).numpy()
    assert np.array_equal(np.isnan(f), np.isnan(tf))
    fin = np.isfinite(tf)
    assert np.array_equal(f[fin], tf[fin])
    # every finite code survives a round trip; +-Inf (e5m2 only) saturates to the largest finite value
    back = oracle.convert(f, oracle.FP32, dt)
    assert np.array_equal(back[fin], codes[fin])
    big = np.array([1e9, -1e9, np.inf, -np.inf, maxv, maxv * 1.5], dtype=np.float32)
    sat = oracle.convert(oracle.convert(big, oracle.FP32, dt), dt, oracle.FP32)
    assert np.array_equal(sat, np.array([maxv, -maxv, maxv, -maxv, maxv, maxv], dtype=np.float32))
    # in-range random values: RNE agrees with torch's cast
    rng = np.random.default_rng(7)
    y = (rng.standard_normal(200000) * (maxv / 8)).astype(np.float32)
    y = y[np.abs(y) < maxv]
    assert np.array_equal(oracle.convert(y, oracle.FP32, dt), torch.from_numpy(y).to(tdt).view(torch.uint8).numpy())


def test_integer_and_bool_pairs_follow_static_cast():
    x = np.array([-3.9, -1.0, -0.5, 0.0, 0.5, 1.0, 2.5, 100.7], dtype=np.float32)
    assert oracle.convert(x, oracle.FP32, oracle.INT32).tolist() == [-3, -1, 0, 0, 0, 1, 2, 100]
    assert oracle.convert(x, oracle.FP32, oracle.BOOLEAN).tolist() == [1, 1, 1, 0, 1, 1, 1, 1]
    i = np.array([-5, 0, 7, 300, 70000, 2 ** 24 + 1], dtype=np.int32)
    assert np.array_equal(oracle.convert(i, oracle.INT32, oracle.FP32), i.astype(np.float32))
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.convert(i, oracle.INT32, oracle.FP16).view(np.uint16), i.astype(np.float64).astype(np.float16).view(np.uint16))
    # int32 -> bf16 is one rounding step from the exact integer (a trip through fp32 would double round this value)
    tricky = np.array([2 ** 30 + 2 ** 22 + 1], dtype=np.int32)
    assert oracle.convert(tricky, oracle.INT32, oracle.BF16).tolist() == [0x4E81]
    assert oracle.convert(np.array([1, 0, 2], dtype=np.uint8), oracle.BOOLEAN, oracle.FP16).view(np.uint16).tolist() == [0x3C00, 0, 0x3C00]


def test_in_place_and_thread_partition_rule():
    x = _c2_like(1_200_000, 3)
    want = oracle.convert(x, oracle.FP32, oracle.FP16)
    buf = x.copy()
    used = oracle.convert_raw(buf.ctypes.data, buf.ctypes.data, oracle.FP32, oracle.FP16, buf.size)
    assert used == 1  # in place with a size change is single threaded (TypeConverter.cpp:929-940)
    assert np.array_equal(buf.view(np.float16)[: x.size].view(np.uint16), want.view(np.uint16))
    out = np.empty(x.size, dtype=np.float16)
    used = oracle.convert_raw(x.ctypes.data, out.ctypes.data, oracle.FP32, oracle.FP16, x.size)
    assert used == min(os.cpu_count() or 1, x.size // 500000)  # TypeConverter.cpp:918
    assert np.array_equal(out.view(np.uint16), want.view(np.uint16))
    # widening in place walks backwards
    h = np.zeros(2 * 1000, dtype=np.float16)
    h[:1000] = np.linspace(-4, 4, 1000).astype(np.float16)
    first = h[:1000].copy()
    oracle.convert_raw(h.ctypes.data, h.ctypes.data, oracle.FP16, oracle.FP32, 1000)
    assert np.array_equal(h.view(np.float32)[:1000], first.astype(np.float32))
