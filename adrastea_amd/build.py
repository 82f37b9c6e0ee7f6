"""Builds libadrastea_kernels_hip.so (the C-ABI library) from csrc/*.hip with hipcc for gfx950.

    python -m adrastea_amd.build            # build if sources are newer than the library
    python -m adrastea_amd.build --force

The library is built in-tree (adrastea_amd/lib/) so that it travels with the source tree to a
GPU machine; nothing is compiled at import time.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libadrastea_kernels_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

SOURCES = ["api.hip", "matmul_general.hip", "gemm_mfma.hip", "gemv_u8.hip", "quantize.hip"]

# packed-fp32 instructions are switched off for all device code (some forms have produced
# wrong results on this hardware generation); the host pass warns that it does not know the
# feature, which is harmless.
CXXFLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-function",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _deps():
    files = [os.path.join(CSRC, f) for f in os.listdir(CSRC)]
    files.append(os.path.join(os.path.dirname(HERE), "include", "adrastea_kernels.h"))
    return files


def is_stale() -> bool:
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    return any(os.path.getmtime(f) > t for f in _deps())


def _compile(src: str) -> str:
    obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *CXXFLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    warn = [l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if warn:
        sys.stderr.write("\n".join(warn) + "\n")
    return obj


def build_library(force: bool = False, extra_flags=()) -> str:
    if not force and not is_stale():
        return LIB
    os.makedirs(LIBDIR, exist_ok=True)
    global CXXFLAGS
    saved = CXXFLAGS
    CXXFLAGS = [*CXXFLAGS, *extra_flags]
    try:
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
            objs = list(ex.map(_compile, SOURCES))
    finally:
        CXXFLAGS = saved
    cmd = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build_library(force="--force" in sys.argv))
