"""Stamps about 380 expressions and backward equations without a GPU (tests/cpp/dry_run_stamp.cpp): planning, source generation and the run-time
compilation for gfx950 run as they do on a GPU box, nothing is launched.  Guards against kernels that do not compile; the
in-process compiler aborts the process on some failures, so the program's output names the case it was working on."""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "dry_run_stamp")


def test_every_planned_kernel_compiles_for_gfx950():
    if not os.path.exists(BINARY):
        subprocess.check_call(["make", "-C", os.path.join(HERE, "cpp"), "dry_run_stamp"])
    result = subprocess.run([BINARY], capture_output=True, text=True, timeout=900)
    tail = "\n".join((result.stdout + result.stderr).splitlines()[-6:])
    assert result.returncode == 0, tail
    assert "0 failures" in result.stdout, tail
