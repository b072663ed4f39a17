"""Runs the C++ API test program (tests/cpp/test_cpp_api.cpp): the same cases the reference spells as gtest suites, written
against this build's C++ headers and linked to the in-tree library."""
from __future__ import annotations

import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "test_cpp_api")


def _binary():
    if not os.path.exists(BINARY):
        subprocess.check_call(["make", "-C", os.path.join(HERE, "cpp")])
    return BINARY


def _run(mode):
    result = subprocess.run([_binary(), mode], capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stdout + result.stderr
    assert "0 failures" in result.stdout


def test_cpp_api_host_cases():
    _run("host")


@pytest.mark.gpu
def test_cpp_api_gpu_cases(gpu):
    _run("gpu")
