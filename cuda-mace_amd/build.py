"""Ahead-of-time build of the gfx950 C-ABI library.

    python cuda-mace_amd/build.py            # compile every source, link cuda_mace/lib/libcuda_mace_hip.so

hipcc cross-compiles for gfx950 without a GPU.  Objects go to cuda-mace_amd/build/ (git-ignored);
the shared library is kept in-tree next to the Python package so that it travels with the source.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "cuda_mace", "lib")
LIB_NAME = "libcuda_mace_hip.so"

SOURCES = ["error.cpp", "mp.hip", "sort.hip", "sh.hip", "geometry.hip", "spline.hip", "linear.hip", "symcon.hip"]

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# Packed-fp32 instruction selection is switched off for every device compile.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if src.endswith(".hip"):
        cmd = [HIPCC, *DEVICE_FLAGS, *COMMON_FLAGS, "-c", path, "-o", obj]
    else:
        cmd = [HIPCC, *COMMON_FLAGS, "-x", "c++", "-c", path, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that is expected.
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    """Compiles all sources (always, even if a library is already there) and links the library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = list(pool.map(_compile, sources))
    out = os.path.join(LIB_DIR, LIB_NAME)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed: %s\n%s" % (" ".join(cmd), res.stderr))
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build()
