"""GPU parity of thorhip_convert (TypeConverter::gpuConvertType) against the CPU oracle, bit for bit."""
import itertools
import json
import os

import numpy as np
import pytest

import oracle
from thor_amd.dtypes import DataType, numpy_carrier, size_of

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
FLOATS = [DataType.fp16, DataType.bf16, DataType.fp8_e4m3, DataType.fp8_e5m2, DataType.fp32, DataType.fp64]
INTS = [DataType.int8, DataType.int16, DataType.int32, DataType.int64, DataType.uint8, DataType.uint16, DataType.uint32,
        DataType.uint64, DataType.boolean]
ALL = FLOATS + INTS
NAN_FREE_COMPARE = {DataType.fp8_e4m3, DataType.fp8_e5m2}


def c2_like(n, seed):
    """BASELINE config 2: N(0,1) with 1% scaled x1e5 (fp16 overflow) and 1% scaled x1e-40 (fp32 subnormals)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(n).astype(np.float32)
    x[0::100] *= np.float32(1e5)
    x[1::100] *= np.float32(1e-40)
    return x


def assert_same_bits(got, want, dtype):
    got_u = got.view(np.dtype(f"u{got.dtype.itemsize}"))
    want_u = want.view(np.dtype(f"u{want.dtype.itemsize}"))
    if dtype in NAN_FREE_COMPARE:
        # fp8 NaN sign/payload is only fixed by the CUDA headers: any NaN code equals any NaN code
        f_got, f_want = oracle.to_f32(got, int(dtype)), oracle.to_f32(want, int(dtype))
        nan = np.isnan(f_want)
        assert np.array_equal(np.isnan(f_got), nan)
        got_u, want_u = got_u[~nan], want_u[~nan]
    bad = np.nonzero(got_u != want_u)[0]
    assert bad.size == 0, f"{bad.size} mismatches, first at {bad[0]}: got {got_u[bad[0]]:#x} want {want_u[bad[0]]:#x}"


@pytest.mark.parametrize("dst", [DataType.fp16, DataType.bf16])
@pytest.mark.parametrize("n", [1, 7, 8, 9, 255, 4097, (1 << 20) + 3])
def test_fp32_narrow_and_back_bit_exact(gpu, dst, n):
    x = c2_like(n, 1235)
    narrow = gpu.convert_array(x, DataType.fp32, dst)
    assert_same_bits(narrow, oracle.convert(x, oracle.FP32, int(dst)), dst)
    back = gpu.convert_array(narrow, dst, DataType.fp32)
    assert_same_bits(back, oracle.convert(narrow, int(dst), oracle.FP32), DataType.fp32)


def test_golden_edge_vectors(gpu):
    with open(os.path.join(GOLDEN, "convert_edges.json")) as f:
        g = json.load(f)
    x = np.array(g["fp32_bits"], dtype=np.uint32).view(np.float32)
    assert np.array_equal(gpu.convert_array(x, DataType.fp32, DataType.fp16).view(np.uint16), np.array(g["fp16_bits"], dtype=np.uint16))
    assert np.array_equal(gpu.convert_array(x, DataType.fp32, DataType.bf16), np.array(g["bf16_bits"], dtype=np.uint16))
    e4 = gpu.convert_array(x, DataType.fp32, DataType.fp8_e4m3)
    e5 = gpu.convert_array(x, DataType.fp32, DataType.fp8_e5m2)
    nan = np.isnan(x)
    assert np.array_equal(e4[~nan], np.array(g["e4m3_bits"], dtype=np.uint8)[~nan])
    assert np.array_equal(e5[~nan], np.array(g["e5m2_bits"], dtype=np.uint8)[~nan])
    assert np.all((e4[nan] & 0x7F) == 0x7F) and np.all((e5[nan] & 0x7F) > 0x7C)


def test_all_16bit_codes_widen_exactly(gpu):
    codes = np.arange(65536, dtype=np.uint16)
    got = gpu.convert_array(codes.view(np.float16), DataType.fp16, DataType.fp32)
    assert_same_bits(got, oracle.convert(codes.view(np.float16), oracle.FP16, oracle.FP32), DataType.fp32)
    got = gpu.convert_array(codes, DataType.bf16, DataType.fp32)
    assert_same_bits(got, oracle.convert(codes, oracle.BF16, oracle.FP32), DataType.fp32)


UNSIGNED = (DataType.uint8, DataType.uint16, DataType.uint32, DataType.uint64)


def _sample_for(src, dst, n, rng):
    """Negative float -> unsigned is undefined in the reference (C++ cast): keep such pairs on non-negative inputs."""
    x = _sample(src, n, rng)
    if dst in UNSIGNED and src not in INTS:
        xf = np.abs(x) if src in (DataType.fp32, DataType.fp64) else np.abs(oracle.to_f32(x, int(src)))
        x = xf if src in (DataType.fp32, DataType.fp64) else oracle.convert(xf.astype(np.float32), oracle.FP32, int(src))
    if dst in UNSIGNED and src in INTS and src != DataType.boolean:
        x = np.abs(x).astype(numpy_carrier(src))
    return x


def _sample(dtype, n, rng):
    """Small, exactly representable magnitudes like the reference's converter test (TypeConverterTest.cpp:10-180) plus
    fractional values so that rounding and truncation are exercised."""
    if dtype == DataType.boolean:
        return rng.integers(0, 2, n).astype(np.uint8)
    if dtype in INTS:
        info = np.iinfo(numpy_carrier(dtype))
        return rng.integers(max(info.min, -100), min(info.max, 100) + 1, n).astype(numpy_carrier(dtype))
    vals = rng.uniform(-20.0, 20.0, n).astype(np.float32)
    vals[::7] = np.round(vals[::7])
    if dtype == DataType.fp32:
        return vals
    if dtype == DataType.fp64:
        return vals.astype(np.float64) + 1e-9
    return oracle.convert(vals, oracle.FP32, int(dtype))


@pytest.mark.parametrize("src,dst", [(s, d) for s, d in itertools.product(ALL, ALL) if s != d])
def test_every_pair_out_of_place(gpu, src, dst):
    rng = np.random.default_rng(int(src) * 100 + int(dst))
    n = 5003
    x = _sample_for(src, dst, n, rng)
    got = gpu.convert_array(x, src, dst)
    want = oracle.convert(x, int(src), int(dst))
    assert_same_bits(got, want, dst)


def wide_integers(src, rng):
    """Integers of every magnitude the type holds: random bits cut to a random width, values one step either side of the ties of a
    24-, 11- and 8-bit significand at every exponent, and the ends of the range."""
    carrier = numpy_carrier(src)
    bits = np.iinfo(carrier).bits
    signed = np.iinfo(carrier).min < 0
    width = rng.integers(1, bits + 1, 20000).astype(np.uint64)
    magnitude = rng.integers(0, 1 << 63, 20000, dtype=np.uint64) * np.uint64(2) + rng.integers(0, 2, 20000).astype(np.uint64)
    magnitude = magnitude >> (np.uint64(64) - width)
    around = []
    for significand in (24, 11, 8):
        for exponent in range(significand, bits):
            tie = (1 << exponent) + (1 << (exponent - significand))  # halfway between two neighbours of that significand
            odd_tie = tie + (1 << (exponent - significand + 1))
            around += [tie - 1, tie, tie + 1, odd_tie - 1, odd_tie, odd_tie + 1, (1 << exponent) - 1, 1 << exponent]
    limit = (1 << (bits - 1)) - 1 if signed else (1 << bits) - 1
    values = np.concatenate([magnitude, np.array([v for v in around if v <= limit], np.uint64), np.array([0, 1, limit], np.uint64)])
    values = np.minimum(values, np.uint64(limit))
    if not signed:
        return values.astype(carrier)
    out = values.astype(np.int64)
    out[::2] = -out[::2]
    out = np.concatenate([out, np.array([np.iinfo(carrier).min], np.int64)])
    return out.astype(carrier)


@pytest.mark.parametrize("src", [DataType.int64, DataType.uint64, DataType.int32, DataType.uint32], ids=lambda d: d.name)
def test_wide_integers_round_once_to_every_float_type(gpu, src):
    """A 64-bit integer becomes fp32 through 32-bit halves with a sticky bit, and a narrower float through a round-to-odd fp32
    image (device code has no 64-bit shift by a register amount, which is what the compiler's expansion of the cast would use): the
    results must be the bits of one round-to-nearest-even step from the integer, at every magnitude and either side of every tie."""
    rng = np.random.default_rng(int(src) + 900)
    x = wide_integers(src, rng)
    for dst in (DataType.fp32, DataType.fp64, DataType.fp16, DataType.bf16, DataType.fp8_e4m3, DataType.fp8_e5m2):
        got = gpu.convert_array(x, src, dst)
        want = oracle.convert(x, int(src), int(dst))
        assert_same_bits(got, want, dst)
        if dst == DataType.fp32:  # and the oracle's rounding against NumPy's own
            np.testing.assert_array_equal(want.view(np.uint32), x.astype(np.float32).view(np.uint32))


@pytest.mark.parametrize("src,dst", [(DataType.fp32, DataType.fp16), (DataType.fp32, DataType.bf16), (DataType.fp16, DataType.fp32),
                                      (DataType.bf16, DataType.fp32), (DataType.fp64, DataType.uint8), (DataType.int8, DataType.fp64),
                                      (DataType.fp32, DataType.int32), (DataType.fp16, DataType.bf16)])
@pytest.mark.parametrize("n", [1, 100, 2048, 2049, 100_003, 1_000_001])
def test_in_place(gpu, src, dst, n):
    from thor_amd.runtime import DeviceBuffer, TypeConverter
    rng = np.random.default_rng(n)
    x = _sample_for(src, dst, n, rng)
    want = oracle.convert(x, int(src), int(dst))
    nbytes = n * max(size_of(src), size_of(dst))
    buf = DeviceBuffer(nbytes + 256)
    guard = np.full(256, 0xA5, dtype=np.uint8)
    buf.upload(guard, offset_bytes=nbytes)
    buf.upload(x)
    TypeConverter.convert_type(buf.ptr, buf.ptr, src, dst, n)
    got = buf.download(numpy_carrier(dst), n)
    assert_same_bits(got, want, dst)
    assert np.array_equal(buf.download(np.uint8, 256, offset_bytes=nbytes), guard), "wrote past the end of the buffer"


def test_no_access_outside_the_range_and_unaligned_views(gpu):
    """The reference's kernels lean on a 128-byte tensor pad; here a ragged tail and an odd base address must stay inside."""
    from thor_amd.runtime import DeviceBuffer, TypeConverter
    n = 10_007
    x = c2_like(n + 3, 5)
    src = DeviceBuffer.from_numpy(x)
    dst = DeviceBuffer((n + 64) * 2)
    dst.memset(0x5A)
    gpu.device_synchronize()
    # element offset 3 on the source (12 bytes: not 16-byte aligned), offset 1 on the destination (2 bytes)
    TypeConverter.convert_type(src.ptr + 12, dst.ptr + 2, DataType.fp32, DataType.fp16, n)
    raw = dst.download(np.uint16, n + 64)
    want = oracle.convert(x[3:3 + n], oracle.FP32, oracle.FP16).view(np.uint16)
    assert np.array_equal(raw[1:1 + n], want)
    assert raw[0] == 0x5A5A and np.all(raw[1 + n:] == 0x5A5A)


@pytest.mark.parametrize("src_off,dst_off", [(1, 1), (3, 3), (2, 1), (0, 3), (1, 0), (5, 5), (7, 2)])
@pytest.mark.parametrize("pair", [("fp32", "fp16"), ("fp16", "fp32"), ("fp32", "bf16"), ("bf16", "fp16"), ("fp16", "fp8_e4m3")], ids=lambda p: "-".join(p))
def test_views_that_begin_inside_a_word(gpu, src_off, dst_off, pair):
    """Source and destination a few elements past a word boundary, by the same count (both become aligned once the slots are
    counted from the boundary below the destination) and by different counts (source words are read where they lie): bit-exact
    against the oracle, guard bytes on both sides of the destination untouched."""
    from thor_amd.runtime import DeviceBuffer, TypeConverter
    src_dtype, dst_dtype = DataType[pair[0]], DataType[pair[1]]
    codes = {"fp32": oracle.FP32, "fp16": oracle.FP16, "bf16": oracle.BF16, "fp8_e4m3": oracle.FP8_E4M3}
    src_code, dst_code = codes[pair[0]], codes[pair[1]]
    dst_carrier = np.dtype(oracle.CARRIER[dst_code])
    n = 70_001
    x32 = c2_like(n + 16, 9)
    x = x32 if pair[0] == "fp32" else oracle.convert(x32, oracle.FP32, src_code)
    src = DeviceBuffer.from_numpy(x)
    dst = DeviceBuffer((n + 64) * dst_carrier.itemsize)
    dst.memset(0x5A)
    gpu.device_synchronize()
    TypeConverter.convert_type(src.ptr + src_off * x.itemsize, dst.ptr + dst_off * dst_carrier.itemsize, src_dtype, dst_dtype, n)
    raw = dst.download(dst_carrier, n + 64)
    want = oracle.convert(x[src_off:src_off + n], src_code, dst_code)
    assert raw[dst_off:dst_off + n].tobytes() == want.tobytes()
    assert np.all(np.frombuffer(raw[:dst_off].tobytes(), np.uint8) == 0x5A) and np.all(np.frombuffer(raw[dst_off + n:].tobytes(), np.uint8) == 0x5A)


def test_overlap_and_argument_errors(gpu):
    from thor_amd._lib import ThorHipError
    from thor_amd.runtime import DeviceBuffer, TypeConverter
    buf = DeviceBuffer(4096)
    with pytest.raises(ThorHipError, match="overlap"):
        TypeConverter.convert_type(buf.ptr, buf.ptr + 8, DataType.fp32, DataType.fp16, 100)
    with pytest.raises(ValueError):
        TypeConverter.convert_type(buf.ptr, buf.ptr, DataType.fp32, DataType.fp32, 100)
    TypeConverter.convert_type(buf.ptr, buf.ptr, DataType.fp32, DataType.fp16, 0)  # empty input is a no-op


def test_full_size_round_trip_properties(gpu):
    """BASELINE config 2 at its full 2^28 elements, checked through size-independent properties: fp16/bf16 -> fp32 -> same
    16-bit type is the identity, and the narrowed stream matches the oracle on strided 2^20-element windows."""
    from thor_amd.runtime import DeviceBuffer, TypeConverter
    n = 1 << 28
    rng = np.random.default_rng(1235)
    block = c2_like(1 << 22, 1235)
    src = DeviceBuffer(n * 4)
    for k in range(n // block.size):
        src.upload(np.roll(block, k * 9973), offset_bytes=k * block.nbytes)
    for dt in (DataType.fp16, DataType.bf16):
        narrow, wide, again = DeviceBuffer(n * 2), DeviceBuffer(n * 4), DeviceBuffer(n * 2)
        TypeConverter.convert_type(src.ptr, narrow.ptr, DataType.fp32, dt, n)
        TypeConverter.convert_type(narrow.ptr, wide.ptr, dt, DataType.fp32, n)
        TypeConverter.convert_type(wide.ptr, again.ptr, DataType.fp32, dt, n)
        for k in (0, 17, 63):
            off = k * block.size
            a = narrow.download(np.uint16, block.size, offset_bytes=off * 2)
            b = again.download(np.uint16, block.size, offset_bytes=off * 2)
            assert np.array_equal(a, b)
            want = oracle.convert(np.roll(block, k * 9973), oracle.FP32, int(dt)).view(np.uint16)
            assert np.array_equal(a, want)
        tail = narrow.download(np.uint16, 1024, offset_bytes=(n - 1024) * 2)
        assert np.array_equal(tail, oracle.convert(np.roll(block, 63 * 9973)[-1024:], oracle.FP32, int(dt)).view(np.uint16))
        for b_ in (narrow, wide, again):
            b_.free()
    src.free()


def test_every_fp32_bit_pattern_narrows_to_bf16_like_the_oracle(gpu):
    """All 2^32 fp32 inputs, 2^26 at a time: the device's fp32 -> bf16 (the hardware conversion, canonical NaN) equals the
    oracle's round-to-nearest-even on every one of them, subnormals, halfway cases, infinities and NaNs included."""
    from thor_amd.runtime import DeviceBuffer, TypeConverter
    n = 1 << 26
    src, dst = DeviceBuffer(n * 4), DeviceBuffer(n * 2)
    for chunk in range(64):
        bits = np.arange(chunk * n, (chunk + 1) * n, dtype=np.uint64).astype(np.uint32)
        src.upload(bits.view(np.float32))
        TypeConverter.convert_type(src.ptr, dst.ptr, DataType.fp32, DataType.bf16, n)
        got = dst.download(np.uint16, n)
        want = oracle.convert(bits.view(np.float32), oracle.FP32, oracle.BF16).view(np.uint16)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, f"chunk {chunk}: {bad.size} mismatches, first input {int(bits[bad[0]]):#010x}: got {got[bad[0]]:#x} want {want[bad[0]]:#x}"
    src.free()
    dst.free()


@pytest.mark.parametrize("n", [3500, 1 << 20, (1 << 24) + 5])
def test_a_kernel_that_follows_sees_the_converted_values(gpu, n):
    """Chains of launches without host synchronisation in between: a buffer that kernels have read is overwritten by a conversion
    and read again by the next launch; every reader must see the newest values (no line of the older contents may survive in
    any cache the streaming stores pass by)."""
    from thor_amd.runtime import DeviceBuffer, Stream, TypeConverter
    stream = Stream(0)
    first, second = c2_like(n, 11), c2_like(n, 12)
    a, b = DeviceBuffer.from_numpy(first, stream), DeviceBuffer.from_numpy(second, stream)
    half, back, again = DeviceBuffer(n * 2), DeviceBuffer(n * 4), DeviceBuffer(n * 2)
    for _ in range(3):
        TypeConverter.convert_type(a.ptr, half.ptr, DataType.fp32, DataType.fp16, n, stream)      # half <- first
        TypeConverter.convert_type(half.ptr, back.ptr, DataType.fp16, DataType.fp32, n, stream)   # readers pull half's lines in
        TypeConverter.convert_type(back.ptr, again.ptr, DataType.fp32, DataType.fp16, n, stream)  # and back's
        TypeConverter.convert_type(b.ptr, half.ptr, DataType.fp32, DataType.fp16, n, stream)      # half <- second, no sync before
        TypeConverter.convert_type(half.ptr, back.ptr, DataType.fp16, DataType.fp32, n, stream)   # must read the second contents
        TypeConverter.convert_type(back.ptr, again.ptr, DataType.fp32, DataType.fp16, n, stream)
        got_back = back.download(np.float32, n, stream)
        got_again = again.download(np.float16, n, stream)
        want_half = oracle.convert(second, oracle.FP32, oracle.FP16)
        assert_same_bits(got_back, oracle.convert(want_half, oracle.FP16, oracle.FP32), DataType.fp32)
        assert_same_bits(got_again, want_half, DataType.fp16)
    for buf in (a, b, half, back, again):
        buf.free()
