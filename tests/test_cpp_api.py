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
    assert "encoded format 3 R 2 flags 4" in out       # 8192 x 2048 under the mi355x policy: one round of 4096 two-row wave64 units
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


@pytest.mark.gpu
def test_cpp_adapter_load_time_path_on_the_device(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    exe = str(tmp_path / "gpu_adapter")
    subprocess.run([hipcc, "-std=c++17", "-O2", "--offload-arch=gfx950", "-I" + os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "cpp", "gpu_adapter.cpp"), "-o", exe, "-L" + LIBDIR, "-lbf16n_hip", "-Wl,-rpath," + LIBDIR],
                   check=True, capture_output=True, timeout=300)
    r = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=120)
    out = r.stdout
    for name in ("output.weight", "blk.0.ffn_gate_exps.weight", "blk.0.ffn_down_shexp.weight"):
        assert f"convert {name} ok" in out, out
    assert "registered 3" in out
    for line in ("lookup ok", "verify ok", "mmv ok", "linear_dense ok", "release ok"):
        assert line in out, out
    assert "invalid_argument bf16n: adapter: the address is not the start of a row" in out
    assert "invalid_argument bf16n: adapter: the tensor overlaps a registered one" in out
    assert "no throw" not in out
    # the reference's log line per converted tensor (patch 0002:324-327)
    assert "roundtrip=OK" in r.stderr and "hufpair" in r.stderr and "nibble" in r.stderr


def test_adapter_registry_on_the_host():
    """Registration, lookup by interior address and release need no device: the registry is host bookkeeping."""
    import ctypes as C

    from orin_qwen_lossless_amd import _lib

    L = _lib.lib()
    assert L.bf16n_adapter_count() == 0
    owner1, owner2 = C.c_int(1), C.c_int(2)
    K, rows = 1024, 64

    def weight(plane):
        w = _lib.Weight()
        w.plane, w.aux, w.format, w.R, w.K, w.rows = plane, 0x7000_0000, 3, 4, K, rows
        return w

    a, b = weight(0x1000_0000), weight(0x1000_0000 + rows * K)       # adjacent tensors of one buffer
    for w, o in ((a, owner1), (b, owner2)):
        _lib.check(L.bf16n_adapter_register(C.byref(w), C.byref(o)))
    got, row0, found = _lib.Weight(), C.c_int64(), C.c_int()
    for addr, want_plane, want_row in ((0x1000_0000, a.plane, 0), (0x1000_0000 + 5 * K, a.plane, 5),
                                       (0x1000_0000 + rows * K, b.plane, 0), (0x1000_0000 + (2 * rows - 1) * K, b.plane, rows - 1)):
        _lib.check(L.bf16n_adapter_lookup(addr, C.byref(got), C.byref(row0), C.byref(found)))
        assert (found.value, got.plane, row0.value) == (1, want_plane, want_row)
    for addr in (0x1000_0000 - K, 0x1000_0000 + 2 * rows * K):
        _lib.check(L.bf16n_adapter_lookup(addr, C.byref(got), C.byref(row0), C.byref(found)))
        assert found.value == 0
    with pytest.raises(ValueError, match="start of a row"):
        _lib.check(L.bf16n_adapter_lookup(0x1000_0000 + 7, C.byref(got), C.byref(row0), C.byref(found)))
    with pytest.raises(ValueError, match="overlaps"):
        c = weight(0x1000_0000 + K)
        _lib.check(L.bf16n_adapter_register(C.byref(c), C.byref(owner1)))
    n = C.c_int()
    _lib.check(L.bf16n_adapter_release(C.byref(owner1), C.byref(n)))
    assert n.value == 1 and L.bf16n_adapter_count() == 1
    _lib.check(L.bf16n_adapter_lookup(0x1000_0000, C.byref(got), C.byref(row0), C.byref(found)))
    assert found.value == 0
    _lib.check(L.bf16n_adapter_release(C.byref(owner2), C.byref(n)))
    assert n.value == 1 and L.bf16n_adapter_count() == 0
    # the loader's tag: 0 stay BF16, 1 NIBBLE, 2 Huffman family (reference engine rules and this build's)
    for engine in (0, 2):
        assert L.bf16n_adapter_choose(248320, 2048, 1, b"hybrid", 8 << 20, 0, engine) == 2
        assert L.bf16n_adapter_choose(512, 2048, 1, b"hybrid", 8 << 20, 0, engine) == 1
        assert L.bf16n_adapter_choose(512, 2048, 256, b"hybrid", 8 << 20, 1, engine) == 2
        assert L.bf16n_adapter_choose(512, 2048, 1, b"huffman", 8 << 20, 0, engine) == 2
        assert L.bf16n_adapter_choose(248320, 2048, 1, b"nibble", 8 << 20, 0, engine) == 1
        assert L.bf16n_adapter_choose(512, 1000, 1, b"hybrid", 8 << 20, 0, engine) == 0


def test_verify_roundtrip_rejects_a_malformed_weight():
    """K = 0 or R = 0 are divisors in the verify step: they must come back as EINVAL, not as a signal."""
    import ctypes as C

    from orin_qwen_lossless_amd import _lib

    L = _lib.lib()
    src = (C.c_uint16 * 1024)()
    ok = C.c_int(-1)
    for K, R, fmt in ((0, 4, 3), (1024, 0, 3), (1024, 0, 2), (1000, 4, 3), (1024, 4, 7)):
        w = _lib.Weight()
        w.plane, w.aux, w.format, w.R, w.K, w.rows = 0x1000, 0x2000, fmt, R, K, 64
        with pytest.raises(ValueError, match="bf16n:"):
            _lib.check(L.bf16n_verify_roundtrip(C.byref(w), src, C.byref(ok)))


@pytest.mark.gpu
def test_standalone_bench_program_runs():
    """The torch-free timing program (csrc/bench_mmv.cpp, built next to the library): a small matrix, the bit-exact
    verify and FP64 check it does before timing, and the read probe's four patterns."""
    import json

    exe = os.path.join(LIBDIR, "bf16n_bench")
    assert os.path.exists(exe), "build it with python -m orin_qwen_lossless_amd.build"
    for extra in ([], ["--tiles", "--rows", "131072", "--K", "1024", "--batch", "3"], ["--f32"]):
        r = subprocess.run([exe, "--rows", "16384", "--reps", "5", "--warm-ms", "5", "--probe"] + extra, check=True,
                           capture_output=True, text=True, timeout=120)
        d = json.loads(r.stdout)
        assert d["max_err_over_sum_abs"] <= 1e-5 and d["median_us"] > 0 and d["GBps"] > 0
        assert all(d[f"read_{p}_w16_GBps"] > 100 for p in ("ranges_nt", "ranges_plain", "stride_nt", "stride_plain"))
