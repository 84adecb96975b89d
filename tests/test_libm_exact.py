"""The restated float routines (glades-ml_amd/csrc/libm_exact.h: tanhf, expm1f, expf, logf as GNU
libc 2.35 computes them) against this machine's C library.  The header is compiled for the host by
g++ here and for the device by hipcc in the product: same source.  The exhaustive comparison over
all 2^32 inputs (`tests/bin/libm_check 1`, half a minute on 8 cores) found no difference; the
committed run visits every 29th float (148 M inputs, every exponent, both signs, NaNs, infinities)
from two starting points."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "bin", "libm_check")
SRC = os.path.join(ROOT, "tests", "libm_check.cpp")


def checker():
    if not os.path.exists(BIN) or os.path.getmtime(BIN) < os.path.getmtime(SRC):
        os.makedirs(os.path.dirname(BIN), exist_ok=True)
        subprocess.check_call(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-fopenmp", "-o", BIN, SRC, "-lm"])
    return BIN


@pytest.mark.parametrize("first", [0, 17])
def test_restated_routines_equal_the_c_library(first):
    out = subprocess.check_output([checker(), "29", str(first)], text=True).split()
    got = dict(zip(out[0::2], (int(v) for v in out[1::2])))
    assert got["inputs"] > 148_000_000
    assert got["tanhf"] == 0 and got["expf"] == 0 and got["logf"] == 0 and got["expm1f"] == 0
