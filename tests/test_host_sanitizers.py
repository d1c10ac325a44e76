"""The host-side decoding of caller-shaped buffers (shapeInfo / TAD logic, stride canonicalisation) compiled with
AddressSanitizer and UndefinedBehaviorSanitizer and run on generated shapes: tests/host_sanitize.cpp.  No GPU."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_shape_and_view_logic_under_sanitizers(tmp_path):
    exe = str(tmp_path / "host_sanitize")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                           "-fno-omit-frame-pointer", os.path.join(HERE, "host_sanitize.cpp"), "-o", exe])
    env = dict(os.environ)
    env["ASAN_OPTIONS"] = "detect_leaks=1:abort_on_error=0:verify_asan_link_order=0"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    out = subprocess.run([exe], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=600)
    text = out.stdout.decode(errors="replace")
    assert out.returncode == 0 and "host sanitize run: ok" in text, text[-3000:]
