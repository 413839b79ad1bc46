"""CPU: the quantiser's fast division path (FMA-based, shared header aiter_amd/csrc/fp8bs_math.h)
compiled for the host and compared exhaustively with IEEE division; also the header's software
e4m3fn conversion against the oracle's.  Host logic only, no GPU."""

import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "host_math", "fastpath_check.cpp")
ORACLE_C = os.path.join(os.path.dirname(HERE), "oracle", "fp8bs_oracle.c")


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("fastpath") / "fastpath_check")
    subprocess.check_call(
        ["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-mfma", "-o", exe, SRC, "-x", "c", ORACLE_C, "-lm"]
    )
    return exe


@pytest.mark.parametrize("mode", ["bf16", "fp16", "cvt"])
def test_fast_division_is_ieee_exact(checker, mode):
    out = subprocess.run([checker, mode], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.startswith("OK")
