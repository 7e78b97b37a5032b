"""Builds ``libcudaBERT.so`` (gfx950) in-tree with hipcc.

    python -m cudabert_amd.build

The library is written next to this file so that the ctypes binding finds it
the way the reference's binding finds its own (cuda_bert/pybert.py:10-12).
hipcc cross-compiles for gfx950 without a GPU being present.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libcudaBERT.so")
SOURCES = ["npy.cc", "weights.cc", "engine.cc", "capi.cc", "gemm.hip", "gemm_bf16_256.hip", "gemm_bf16_128.hip", "attention.hip", "rowwise.hip", "noalloc.hip"]

# -packed-fp32-ops is switched off: the compiler must not form packed FP32 math.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result", "-Wno-unknown-attributes",
                "-Wno-unused-command-line-argument"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _compile(src: str, objdir: str, extra) -> str:
    obj = os.path.join(objdir, os.path.basename(src) + ".o")
    cmd = [hipcc(), "-c", os.path.join(CSRC, src), "-o", obj] + COMMON_FLAGS + list(extra)
    if src.endswith(".hip"):
        cmd += DEVICE_FLAGS
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj


def build_library(verbose: bool = True, extra_flags=()) -> str:
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, objdir, extra_flags), SOURCES))
    tmp = LIB + ".tmp"
    cmd = [hipcc(), "-shared", "-o", tmp] + objs + DEVICE_FLAGS + ["-Wl,-soname,libcudaBERT.so"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    os.replace(tmp, LIB)
    if verbose:
        print("built", LIB, "(%d KiB)" % (os.path.getsize(LIB) // 1024))
    return LIB


if __name__ == "__main__":
    build_library(extra_flags=sys.argv[1:])
