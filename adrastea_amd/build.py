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

SOURCES = ["api.hip", "matmul_general.hip", "gemm_mfma.hip", "gemv_u8.hip", "quantize.hip",
           "softmax.hip", "attention.hip", "error_stats.hip", "microbench.hip", "gemv_f16.hip",
           "device.hip"]

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


STAMPS_LIB = os.path.join(LIBDIR, "libadrastea_kernels_hip_stamps.so")


def build_stamps_library(force: bool = False) -> str:
    """The diagnostic twin of the library: gemm_mfma.hip compiled with -DADR_PHASE_STAMPS (its tiled
    GEMM kernels then leave per-wavefront time stamps of prologue / K loop / epilogue in the
    buffer passed as workspace), linked with the other objects of build_library().  Read by
    `bench.py --phase-stamps`; nothing else loads it."""
    build_library(force=False)
    if (not force and os.path.exists(STAMPS_LIB)
            and all(os.path.getmtime(f) <= os.path.getmtime(STAMPS_LIB) for f in _deps())):
        return STAMPS_LIB
    obj = os.path.join(LIBDIR, "gemm_mfma_stamps.o")
    cmd = [HIPCC, *CXXFLAGS, "-DADR_PHASE_STAMPS", "-c", os.path.join(CSRC, "gemm_mfma.hip"), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for the stamps build:\n{r.stdout}\n{r.stderr}")
    objs = [os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o") for src in SOURCES if src != "gemm_mfma.hip"]
    cmd = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", STAMPS_LIB, obj, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return STAMPS_LIB


# Code objects for an unmodified host of the reference: module name -> source.  Each exports the
# device symbols that host looks up in its module of that name, with the same kernel arguments.
LEGACY_DIR = os.path.join(LIBDIR, "legacy")
LEGACY_MODULES = {"matmul.co": "legacy_matmul.hip", "error_stats.co": "legacy_error_stats.hip"}


def build_legacy_modules(force: bool = False) -> list:
    """hipcc --genco of the legacy-symbol code objects into lib/legacy/."""
    os.makedirs(LEGACY_DIR, exist_ok=True)
    outs = []
    for name, src in LEGACY_MODULES.items():
        out = os.path.join(LEGACY_DIR, name)
        outs.append(out)
        if (not force and os.path.exists(out)
                and all(os.path.getmtime(f) <= os.path.getmtime(out) for f in _deps())):
            continue
        flags = [f for f in CXXFLAGS if f != "-fPIC"]
        cmd = [HIPCC, "--genco", *flags, os.path.join(CSRC, src), "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc --genco failed for {src}:\n{r.stdout}\n{r.stderr}")
    return outs


HOST_TEST_SRC = os.path.join(os.path.dirname(HERE), "tests", "cpp", "test_host.cpp")
HOST_TEST_BIN = os.path.join(os.path.dirname(HERE), "tests", "cpp", "bin", "test_host")


def build_host_test(force: bool = False) -> str:
    """Compiles the C++ host-side test (header-only host/*.hpp over the C ABI) with g++."""
    deps = [HOST_TEST_SRC, LIB] + [os.path.join(HERE, "host", f) for f in os.listdir(os.path.join(HERE, "host"))]
    if (not force and os.path.exists(HOST_TEST_BIN)
            and all(os.path.getmtime(d) <= os.path.getmtime(HOST_TEST_BIN) for d in deps)):
        return HOST_TEST_BIN
    os.makedirs(os.path.dirname(HOST_TEST_BIN), exist_ok=True)
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-o", HOST_TEST_BIN, HOST_TEST_SRC, "-L" + LIBDIR,
           "-ladrastea_kernels_hip", "-ldl", "-Wl,-rpath,$ORIGIN/../../../adrastea_amd/lib",
           "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"g++ failed for the host test:\n{r.stdout}\n{r.stderr}")
    return HOST_TEST_BIN


if __name__ == "__main__":
    print(build_library(force="--force" in sys.argv))
    print(build_stamps_library(force="--force" in sys.argv))
    print(build_legacy_modules(force="--force" in sys.argv))
    print(build_host_test(force="--force" in sys.argv))
