"""The C++ API headers (include/bf16n/*.h, the reference's core/include/bf16n/{encode,policy,launch}.h restated over
the C ABI) compile against the library and translate status codes into the reference's exception types."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "orin_qwen_lossless_amd")


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_cpp_headers_compile_and_run(tmp_path):
    from orin_qwen_lossless_amd import _lib

    _lib.lib()  # the library must be built
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    exe = str(tmp_path / "api_smoke")
    subprocess.run([hipcc, "-std=c++17", "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "cpp", "api_smoke.cpp"),
                    "-o", exe, "-L" + LIBDIR, "-lbf16n_hip", "-Wl,-rpath," + LIBDIR], check=True, capture_output=True, timeout=300)
    out = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=60).stdout.splitlines()
    got = {ln.split()[0]: ln.split(None, 1)[1] if " " in ln else "" for ln in out}
    assert got["choose_bad_k"] == "0"
    assert got["choose_llama"] == "3 16 0 0"      # reference: dense HUFPAIR, largest R leaving >= 512 units
    assert got["choose_mi355x"] == "3 16 0 1"
    assert got["encode"] == "16384 3 4 1 1024 0"
    assert got["encode_wave64"] == "4"
    assert got["invalid_argument"].startswith("bf16n encode:")
    assert "no_throw" not in got
    assert any("fragment" in ln for ln in out if ln.startswith("invalid_argument"))
    assert got["views"] == "8 1"


@pytest.mark.gpu
def test_cpp_api_on_the_device(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    exe = str(tmp_path / "gpu_mmv")
    subprocess.run([hipcc, "-std=c++17", "-O2", "--offload-arch=gfx950", "-I" + os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "gpu_mmv.cpp"), "-o", exe, "-L" + LIBDIR, "-lbf16n_hip", "-Wl,-rpath," + LIBDIR],
                   check=True, capture_output=True, timeout=300)
    out = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=120).stdout
    assert "encoded format 3 R 4 flags 4" in out       # 4096 x 2048 under the mi355x policy: wave64 units of 4 rows
    assert "dequant ok" in out and "mmv ok" in out
    assert "invalid_argument bf16n: dequant rows must be whole units" in out


@pytest.mark.gpu
def test_cpp_api_moe_layer_on_the_device(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    exe = str(tmp_path / "gpu_moe")
    subprocess.run([hipcc, "-std=c++17", "-O2", "--offload-arch=gfx950", "-I" + os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "gpu_moe.cpp"), "-o", exe, "-L" + LIBDIR, "-lbf16n_hip", "-Wl,-rpath," + LIBDIR],
                   check=True, capture_output=True, timeout=300)
    out = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=120).stdout
    assert "experts R 32 32 flags 4 4" in out          # the mi355x policy: 32 x 256 tiles for experts
    assert "mm_ids_supported 1 1" in out
    assert "batched ok" in out and "gemv ok" in out, out
