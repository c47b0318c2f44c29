"""Builds libqmm_hip.so (the gfx950 kernels + the C ABI) with hipcc, in-tree.

    python -m metaljax_amd.build            the library (and the PJRT plugin)
    python -m metaljax_amd.build --probe    libqmm_probe.so only (bench.py --probe)
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
    return LIB


PROBE_LIB = os.path.join(LIBDIR, "libqmm_probe.so")


def build_probe(verbose: bool = False) -> str:
    """The measuring kernels of `bench.py --probe` (read-only and empty
    launches), a library of their own: not part of the quantized-matmul ABI and
    not built by default (`python -m metaljax_amd.build --probe`)."""
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = ["hipcc", *FLAGS, "-shared", os.path.join(CSRC, "probe_stream.hip"), "-o", PROBE_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError(f"hipcc failed on probe_stream.hip:\n{r.stderr}")
    if verbose:
        print(f"built {PROBE_LIB}")
    return PROBE_LIB


PJRT_LIB = os.path.join(LIBDIR, "libqmm_pjrt.so")
PJRT_HARNESS = os.path.join(LIBDIR, "libqmm_pjrt_harness.so")


def pjrt_header_dir():
    """The directory holding OpenXLA's `pjrt_c_api.h`: $PJRT_C_API_INCLUDE, or
    the reference checkout's vendored copy; None when there is none."""
    for d in (os.environ.get("PJRT_C_API_INCLUDE"), "/root/reference/plugin/vendor"):
        if d and os.path.exists(os.path.join(d, "pjrt_c_api.h")):
            return d
    return None


def build_pjrt(verbose: bool = False):
    """The PJRT plugin (`GetPjrtApi` over `metaljax_amd.engine`) and the C++
    harness the tests drive it with.  Host code only.  Both are compiled against
    the header where it lies (it is not part of this tree); without the header
    the step is skipped and what is already built stays."""
    inc = pjrt_header_dir()
    if inc is None:
        if verbose:
            print("pjrt_c_api.h not found (PJRT_C_API_INCLUDE): PJRT plugin not rebuilt")
        return None
    import sysconfig
    os.makedirs(LIBDIR, exist_ok=True)
    base = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wno-unused-function", "-I", inc]
    # the Python symbols resolve against the process that loads the plugin
    # (a Python interpreter), so it is not linked against libpython
    jobs = [(base + ["-I", sysconfig.get_paths()["include"], os.path.join(CSRC, "pjrt_plugin.cc"), "-o", PJRT_LIB], PJRT_LIB),
            (base + [os.path.join(os.path.dirname(HERE), "tests", "pjrt_harness.cc"), "-ldl", "-o", PJRT_HARNESS], PJRT_HARNESS)]
    for cmd, out in jobs:
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode:
            raise RuntimeError(f"g++ failed on {out}:\n{r.stderr}")
        if verbose:
            print(f"built {out}")
    return PJRT_LIB


if __name__ == "__main__":
    if "--probe" in sys.argv[1:]:
        build_probe(verbose=True)
    else:
        build(verbose=True)
        build_pjrt(verbose=True)
