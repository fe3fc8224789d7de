"""Builds ``libcct_hip.so`` (the gfx950 driver library) in-tree with hipcc.

The library holds gfx950 code objects only.  Sources live in ``csrc/``; the public C ABI is
``include/cct_hip.h`` at the repository root.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "libcct_hip.so")
SOURCES = ["api.hip", "lower.hip", "lift.hip", "gemm.hip", "fc_small.hip", "conv_small.hip", "direct.hip", "strided.hip", "eltwise.hip", "corpus.hip", "bridge_capi.cpp"]

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # never let the compiler form packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _compile(src):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, "-x", "hip"] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj


def build_library(verbose=True):
    """Compile every source for gfx950 and link the shared library.  Always recompiles."""
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", LIB, file=sys.stderr)
    return LIB


if __name__ == "__main__":
    build_library()
