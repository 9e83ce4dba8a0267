"""Builds librbmoe.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m rustingbrain_amd.build          # compile every source, link the library

The packed-FP32 target feature is switched off for all device code, and floating
point contraction is off so that only the fused multiply-adds written in the
sources exist (the router's arithmetic order is part of the routing contract).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "librbmoe.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


# Extra compiler flags for experiments with the kernels' compile-time shapes, e.g.
#   RBMOE_HIPCC_EXTRA="-DRBMOE_STREAM_NW=8 -DRBMOE_STREAM_OCC=1" python -m rustingbrain_amd.build
# (eight waves share one activation slice); read here, never by the library.
FLAGS += os.environ.get("RBMOE_HIPCC_EXTRA", "").split()


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, src[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(jobs: int = 4) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    build_bench()
    build_host()
    return LIB


BENCH_SRC = os.path.join(CSRC, "bench", "rbmoe_bench.hip")
BENCH_LIB = os.path.join(HERE, "librbmoe_bench.so")


def build_bench() -> str:
    """The benchmark's measurement helpers (include/rbmoe_bench.h): a library of their own, not part of librbmoe.so."""
    cmd = [HIPCC, *FLAGS, "-shared", BENCH_SRC, "-o", BENCH_LIB]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("bench helper build failed:\n" + res.stderr)
    return BENCH_LIB


HOST = os.path.join(HERE, "host")
TUTORIAL = os.path.join(HOST, "moe_tutorial")


def build_host() -> str:
    """The C++ host mirror's driver (rustingbrain_amd/host/moe_tutorial), linked against librbmoe.so."""
    cmd = ["g++", "-O2", "-std=c++17", "-Wall", os.path.join(HOST, "moe_tutorial.cpp"), "-o", TUTORIAL,
           "-L" + HERE, "-lrbmoe", "-Wl,-rpath,$ORIGIN/.."]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("host build failed:\n" + res.stderr)
    return TUTORIAL


if __name__ == "__main__":
    print(build())
