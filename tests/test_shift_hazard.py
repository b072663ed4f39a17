"""MI355X computes a 64-bit vector shift (v_lshlrev_b64, v_lshrrev_b64, v_ashrrev_i64) wrong, silently and about one time in ten,
when the shift amount is in the last vector register the wavefront owns (measured with an inline-assembly probe: 384 562 396 wrong
results of 4 194 304 000 with the amount in v15 of 16 registers, none with v16 owned as well).  The compiler of this toolchain avoids
that placement for gfx90a only, and its expansion of a 64-bit integer -> fp32 cast contains such a shift.  The device code of this
library therefore has no 64-bit shift by a register amount at all; kernels compiled at run time are scanned as they are loaded
(CompiledEquation.cpp refuses one that has it), and this test scans the kernels that are compiled ahead of time into the library."""
from __future__ import annotations

import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY = os.path.join(os.path.dirname(HERE), "thor_amd", "libthor_amd.so")


def shifts_of(words):
    """(amount operand of every 64-bit vector shift in a stream of little-endian dwords): VOP3 encoding, first dword
    [31:16] = 0xD28F / 0xD290 / 0xD291 with no modifier bits, second dword [8:0] = amount, [31:18] = 0."""
    first, second = words[:-1], words[1:]
    opcode = first >> 16
    hit = ((opcode == 0xD28F) | (opcode == 0xD290) | (opcode == 0xD291)) & ((first & 0xFF00) == 0) & ((second >> 18) == 0)
    return second[hit] & 0x1FF


def test_the_scan_reads_the_encoding_the_assembler_writes():
    # v_lshlrev_b64 v[6:7], v63, -1 / v_lshrrev_b64 v[10:11], v6, -1 / v_ashrrev_i64 v[2:3], v7, v[4:5] / v_lshlrev_b64 v[2:3], 2, v[4:5]
    stream = bytes([0x06, 0x00, 0x8f, 0xd2, 0x3f, 0x83, 0x01, 0x00, 0x0a, 0x00, 0x90, 0xd2, 0x06, 0x83, 0x01, 0x00,
                    0x02, 0x00, 0x91, 0xd2, 0x07, 0x09, 0x02, 0x00, 0x02, 0x00, 0x8f, 0xd2, 0x82, 0x08, 0x02, 0x00])
    amounts = shifts_of(np.frombuffer(stream, "<u4"))
    assert amounts.tolist() == [256 + 63, 256 + 6, 256 + 7, 0x82]


def test_no_ahead_of_time_kernel_shifts_64_bits_by_a_vector_register():
    raw = np.fromfile(LIBRARY, dtype=np.uint8)
    amounts = shifts_of(raw[:raw.size // 4 * 4].view("<u4"))
    assert amounts.size > 100, "the library's gfx950 code is expected to be stored uncompressed (shifts by constants were always found)"
    in_registers = amounts[amounts >= 256] - 256
    assert in_registers.size == 0, f"64-bit vector shifts by register amounts: v{sorted(set(in_registers.tolist()))}"


def u64_to_f32_through_halves(values):
    """The steps of the device's u64ToF32 (thorhip_numeric.h), one NumPy operation per device operation: the high half normalised
    with 32-bit shifts, the bits that do not fit 32 folded into a sticky bit, one rounding 32-bit conversion, exact scaling."""
    values = np.asarray(values, np.uint64)
    hi, lo = (values >> np.uint64(32)).astype(np.uint32), (values & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    lz = np.where(hi == 0, 0, 31 - np.floor(np.log2(np.maximum(hi, 1).astype(np.float64))).astype(np.int64)).astype(np.uint32)
    shifted_in = np.where(lz == 0, np.uint32(0), lo >> (np.uint32(32) - np.maximum(lz, 1)).astype(np.uint32))
    top = ((hi << lz) | shifted_in).astype(np.uint32)
    rest = (lo << lz).astype(np.uint32)
    rounded = (top | (rest != 0).astype(np.uint32)).astype(np.float32)  # uint32 -> float32 rounds to nearest even
    wide = np.ldexp(rounded, (32 - lz.astype(np.int64)).astype(np.int32)).astype(np.float32)
    return np.where(hi == 0, lo.astype(np.float32), wide)


def test_the_conversion_through_32_bit_halves_rounds_like_the_cast():
    rng = np.random.default_rng(5)
    width = rng.integers(1, 65, 200000).astype(np.uint64)
    random = (rng.integers(0, 1 << 63, 200000, dtype=np.uint64) * np.uint64(2) + rng.integers(0, 2, 200000).astype(np.uint64)) >> (np.uint64(64) - width)
    ties = [(1 << e) + (k << (e - 24)) + d for e in range(24, 64) for k in (1, 3, 5, 7) for d in (-1, 0, 1) if (1 << e) + (k << (e - 24)) + d < (1 << 64)]
    edges = [0, 1, (1 << 24) - 1, 1 << 24, (1 << 32) - 1, 1 << 32, (1 << 32) + 1, (1 << 63), (1 << 64) - 1, (1 << 64) - (1 << 39), (1 << 64) - (1 << 39) - 1]
    values = np.concatenate([random, np.array(ties + edges, np.uint64)])
    np.testing.assert_array_equal(u64_to_f32_through_halves(values).view(np.uint32), values.astype(np.float32).view(np.uint32))
