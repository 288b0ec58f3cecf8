"""Builds libhot_gfx950.so (the C-ABI library with the gfx950 kernels) in-tree.

    python -m hot_amd.build                 # everything
    python -m hot_amd.build gemm_i8.hip     # recompile one source, relink

hipcc cross-compiles for gfx950 without a GPU.  Packed-FP32 instruction
selection is switched off for all device code.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhot_gfx950.so")
SOURCES = ["hq_rowwise.hip", "colwise.hip", "hla_big.hip", "gemm_i8.hip", "backward.hip", "ceilings.hip", "hla_expand.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",   # the direct-to-LDS loads name m0 as clobbered; clang remarks on it at every use
    # the column-wise kernels hold a whole token block in registers: their loops must unroll fully
    "-mllvm", "-pragma-unroll-threshold=1000000",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libhot_gfx950.so cannot be built")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [_hipcc(), *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the AMDGPU feature name and says so; drop that line
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True, only=None) -> str:
    """Compiles every source and links the library.  `only` (a list of source names) recompiles just
    those and reuses the other object files of an earlier full build: a developer shortcut."""
    todo = [s for s in SOURCES if not only or s in only
            or not os.path.exists(os.path.join(CSRC, s.replace(".hip", ".o")))]
    with ThreadPoolExecutor(max_workers=min(6, len(SOURCES))) as ex:
        list(ex.map(_compile, todo))
    objs = [os.path.join(CSRC, s.replace(".hip", ".o")) for s in SOURCES]
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(only=[a for a in sys.argv[1:] if a.endswith(".hip")] or None)
