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
