"""Builds libbf16n_hip.so (host encoder/policy + C ABI + HIP kernels for gfx950) in-tree with hipcc.

python -m orin_qwen_lossless_amd.build            # compile what changed
The library sits next to this file so that it travels with the source tree; nothing is installed."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libbf16n_hip.so")
BENCH = os.path.join(HERE, "bf16n_bench")  # stand-alone timing program (csrc/bench_mmv.cpp), linked against the library
PROBE = os.path.join(HERE, "libbf16n_probe.so")  # read-bandwidth probe (csrc/bench_probe.hip): measurement only, loaded by the benchmarks
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

SOURCES = ["encode.cpp", "policy.cpp", "capi.cpp", "adapter.cpp", "dense.cpp", "kernels_compat.hip", "kernels_w64.hip", "kernels_moe.hip", "kernels_mm_ids.hip", "kernels_tile.hip"]
COMMON = ["-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-Wall", "-Wno-unused-function"]
HIP_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src: str, force: bool) -> str:
    path = os.path.join(CSRC, src)
    obj = os.path.join(OBJ, src + ".o")
    deps = [path] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")] + [
        os.path.join(ROOT, "include", "bf16n_c.h"), os.path.join(ROOT, "include", "bf16n", "format.h")]
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) >= os.path.getmtime(d) for d in deps):
        return obj
    cmd = [HIPCC] + COMMON + (HIP_FLAGS if src.endswith(".hip") else ["-x", "hip"] + HIP_FLAGS if src == "adapter.cpp" else ["-x", "hip", "--offload-arch=gfx950"] if src == "capi.cpp"
                             else ["-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include"] if src == "dense.cpp" else []) + ["-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout + r.stderr)
        raise RuntimeError(f"hipcc failed on {src}")
    return obj


def build(force: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        r = subprocess.run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs + ["-lpthread", "-ldl"], capture_output=True, text=True)
        if r.returncode != 0:
            sys.stderr.write(r.stdout + r.stderr)
            raise RuntimeError("link failed")
    probe_src = os.path.join(CSRC, "bench_probe.hip")
    if force or not os.path.exists(PROBE) or os.path.getmtime(PROBE) < os.path.getmtime(probe_src):
        r = subprocess.run([HIPCC] + COMMON + HIP_FLAGS + ["-shared", probe_src, "-o", PROBE], capture_output=True, text=True)
        if r.returncode != 0:
            sys.stderr.write(r.stdout + r.stderr)
            raise RuntimeError("building libbf16n_probe.so failed")
    bench_src = os.path.join(CSRC, "bench_mmv.cpp")
    if force or not os.path.exists(BENCH) or os.path.getmtime(BENCH) < max(os.path.getmtime(bench_src), os.path.getmtime(LIB), os.path.getmtime(PROBE)):
        r = subprocess.run([HIPCC, "-O2", "-std=c++17", "-x", "hip", "--offload-arch=gfx950", "-I" + os.path.join(ROOT, "include"), bench_src,
                            "-o", BENCH, "-L" + HERE, "-lbf16n_hip", "-lbf16n_probe", "-Wl,-rpath,$ORIGIN", "-lpthread"], capture_output=True, text=True)
        if r.returncode != 0:
            sys.stderr.write(r.stdout + r.stderr)
            raise RuntimeError("building bf16n_bench failed")
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
