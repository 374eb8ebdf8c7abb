"""The host encoder and the shape policy built with AddressSanitizer and UBSan (g++, no GPU code) and driven through
every format and layout: memory errors and undefined behaviour in the load-time path fail this test."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "orin_qwen_lossless_amd", "csrc")


@pytest.mark.skipif(shutil.which("g++") is None, reason="no g++")
def test_host_encoder_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "host_sanitize")
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                    "-static-libasan", "-static-libubsan",
                    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, os.path.join(ROOT, "tests", "cpp", "host_sanitize.cpp"),
                    os.path.join(CSRC, "encode.cpp"), os.path.join(CSRC, "policy.cpp"), "-o", exe, "-lpthread"],
                   check=True, capture_output=True, timeout=600)
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "fallback format 2, tiles 2 R 16" in r.stdout
    assert "thrown 6" in r.stdout and "encoded " in r.stdout
