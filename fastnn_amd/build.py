"""Builds libfastnn_hip.so (hand-written HIP kernels for gfx950 + the C ABI) in-tree.

    python -m fastnn_amd.build [--force]

hipcc cross-compiles for gfx950 without a GPU.  The library is written next to this file
so that it travels with the source tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libfastnn_hip.so")

HIP_SOURCES = ["api.hip", "qgemv.hip", "qgemm_generic.hip", "qgemm_tiled.hip", "qgemm_i8.hip", "qgemm_digits.hip", "qgemv_mfma.hip", "qgemv_i8dot.hip", "qgemv_rows16.hip", "i8act.hip", "qconv.hip", "qconv_float.hip", "qconv_implicit.hip", "eltwise.hip",
               "qgemm_stream.hip", "qgemm_stream_i8.hip", "qgemm_stream_i4.hip", "qgemm_stream_u4.hip", "qgemm_stream_u8.hip",
               "qgemm_stream_f8.hip", "qgemm_stream_f8r.hip", "qgemm_stream_f4.hip", "qgemm_stream_i4cb.hip"]
HOST_SOURCES = ["quantize_host.cpp", "hip_backend.cpp"]

# -ffp-contract=off: the integer/quantisation formulas must evaluate exactly as written;
# hot loops ask for fused multiply-adds explicitly.  Packed-FP32 instructions are disabled.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-Wall", "-pthread"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = False, verbose: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(os.path.dirname(HERE), "include", "fastnn_hip.h"))
    headers.append(os.path.join(os.path.dirname(HERE), "include", "fastnn_hip_backend.h"))
    headers = [h for h in headers if os.path.exists(h)]
    hipcc = _hipcc()
    jobs = []
    objs = []
    for src in HIP_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ, src + ".o")
        objs.append(o)
        if force or _stale(o, [s] + headers):
            jobs.append([hipcc] + HIP_FLAGS + ["-c", s, "-o", o])
    for src in HOST_SOURCES:
        s = os.path.join(CSRC, src)
        if not os.path.exists(s):
            continue
        o = os.path.join(OBJ, src + ".o")
        objs.append(o)
        if force or _stale(o, [s] + headers):
            jobs.append(["g++"] + HOST_FLAGS + ["-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__", "-c", s, "-o", o])
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for out in ex.map(_run, jobs):
            if verbose and out.strip():
                print(out)
    if jobs or force or not os.path.exists(LIB):
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-lpthread"])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
