"""Routines of the device's float arithmetic that are written so that a host compiler builds them to the same bits
(fused multiply-adds and integer operations only), checked on the host against the C library the reference evaluates.

The Tanh transform below 1: tests/tanh_host_check.cpp builds libnd4j_amd/csrc/tanh_poly.h, the lines
the device compiles (fused multiply-adds only, so the bits agree), and compares every 61st float in (0, 1) with the C
library's tanhf, which is what the reference evaluates (include/templatemath.h:847, include/ops/ops.h:1362).  Over ALL
floats below 1 (``tanh_host_check 1``, a minute and a half on one core) the histogram is 1006738843 / 58222902 / 391470
at 0 / 1 / 2 ULP from tanhf and none further; 1064279766 / 1073449 at 0 / 1 ULP from the correctly rounded value.

The Log transform: tests/log_host_check.cpp builds libnd4j_amd/csrc/log_poly.h and compares every 127th positive float with
logf (include/templatemath.h, include/ops/ops.h: simdOps::Log).  Over ALL 2139095039 positive floats, denormals included
(``log_host_check 1``), 2066666777 are identical with logf and 72428262 at 1 ULP, none further; 2066792322 / 72302717 at
0 / 1 ULP from the correctly rounded value."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_tanh_polynomial_within_two_ulp_of_the_c_library(tmp_path):
    exe = str(tmp_path / "tanh_host_check")
    # no contraction of the two plain products into neighbouring operations: the device does not contract them either
    subprocess.check_call(["g++", "-std=c++17", "-O2", "-ffp-contract=off", os.path.join(HERE, "tanh_host_check.cpp"), "-o", exe])
    out = subprocess.run([exe, "61"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=300)
    text = out.stdout.decode(errors="replace")
    assert out.returncode == 0 and "tanh host check: ok" in text, text


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_log_routine_within_one_ulp_of_the_c_library(tmp_path):
    exe = str(tmp_path / "log_host_check")
    subprocess.check_call(["g++", "-std=c++17", "-O2", "-ffp-contract=off", os.path.join(HERE, "log_host_check.cpp"), "-o", exe])
    out = subprocess.run([exe, "127"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=300)
    text = out.stdout.decode(errors="replace")
    assert out.returncode == 0 and "log host check: ok" in text, text
