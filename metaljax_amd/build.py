"""Builds libqmm_hip.so (the gfx950 kernels + the C ABI) with hipcc, in-tree.

    python -m metaljax_amd.build
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libqmm_hip.so")
SOURCES = ["qmm_api.hip", "qmm_gemv.hip", "qmm_skinny.hip", "qmm_skinny2.hip", "qmm_gemm.hip", "qmm_gemm2.hip", "qmm_gemm2s.hip", "qmm_mxfp4.hip", "qmm_util.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function"]


def _compile(src: str) -> str:
    obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")
    # QMM_EXPERIMENTS=1: a measuring build whose kernel choice can be overridden
    # through QMM_* environment switches; the normal build reads no environment
    extra = ["-DQMM_EXPERIMENTS"] if os.environ.get("QMM_EXPERIMENTS") == "1" else []
    if os.environ.get("QMM_TIMELINE") == "1":       # clock stamps in the decode kernel (qmm_debug_stamps)
        extra.append("-DQMM_TIMELINE")
    cmd = ["hipcc", *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = False) -> str:
    """Compile every kernel source for gfx950 and link the shared library."""
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    build_probe(verbose)
    return LIB


PROBE_LIB = os.path.join(LIBDIR, "libqmm_probe.so")


def build_probe(verbose: bool = False) -> str:
    """The measuring kernels of `bench.py --probe` (read-only and empty
    launches), a library of their own: not part of the quantized-matmul ABI."""
    cmd = ["hipcc", *FLAGS, "-shared", os.path.join(CSRC, "probe_stream.hip"), "-o", PROBE_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f"hipcc failed on probe_stream.hip:\n{r.stderr}")
    if verbose:
        print(f"built {PROBE_LIB}")
    return PROBE_LIB


if __name__ == "__main__":
    build(verbose=True)
