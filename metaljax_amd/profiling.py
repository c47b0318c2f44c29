"""Turns a rocprofv3 kernel-trace database into the short text summary kept
under profiles/.

    rocprofv3 --kernel-trace -d OUT -o run -- python3 bench.py ...
    python -m metaljax_amd.profiling OUT > profiles/<kernel>_<workload>.txt
"""

from __future__ import annotations

import glob
import sqlite3
import sys


def kernel_stats(path: str):
    """Rows (kernel, grid, block, calls, avg_ns, min_ns, max_ns, total_ns) per kernel name."""
    dbs = [path] if path.endswith(".db") else glob.glob(path + "/**/*.db", recursive=True)
    rows = []
    for dbp in dbs:
        cur = sqlite3.connect(dbp).cursor()
        q = ("select name, grid_x * grid_y * grid_z, workgroup_x, count(*), avg(duration), "
             "min(duration), max(duration), sum(duration) from kernels "
             "group by name, grid_x, grid_y, workgroup_x order by sum(duration) desc")
        rows += cur.execute(q).fetchall()
    return rows


def counter_stats(path: str):
    """Rows (kernel, counter, mean value per dispatch, dispatches)."""
    dbs = [path] if path.endswith(".db") else glob.glob(path + "/**/*.db", recursive=True)
    rows = []
    for dbp in dbs:
        cur = sqlite3.connect(dbp).cursor()
        try:
            rows += cur.execute("select kernel_name, counter_name, avg(value), count(*) from "
                                "counters_collection group by kernel_name, counter_name").fetchall()
        except sqlite3.Error:
            pass
    return rows


def _short(name: str) -> str:
    name = name.replace("(anonymous namespace)::", "")
    if name.startswith("void "):
        name = name[5:]
    if name.startswith("qmm::"):
        name = name[5:]
    return name.split("(")[0][:64]


def stream_probe(nbytes: int = 32 << 20, reps: int = 400):
    """What a single launch reaches on this GPU whatever its arithmetic: the
    per-launch time (HIP events around a graph replay, like the benchmark's
    decode leg) of read-only launches over `nbytes` in several geometries, each
    cycling through distinct buffers of more than twice the last-level cache
    so that every launch streams from HBM, and of empty launches of the decode
    kernel's geometry.  Returns a dict of results."""
    import ctypes
    import os

    import torch
    here = os.path.dirname(os.path.abspath(__file__))
    path = os.path.join(here, "lib", "libqmm_probe.so")
    if not os.path.exists(path):
        raise RuntimeError("libqmm_probe.so is not built: run `python -m metaljax_amd.build --probe`")
    lib = ctypes.CDLL(path)
    vp, ci, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
    lib.probe_read.argtypes = [vp, i64, vp, ci, ci, ci, ci, vp]
    lib.probe_empty.argtypes = [vp, ci, ci, ci, vp]
    n_sets = (2 * (256 << 20)) // nbytes + 1
    bufs = [torch.randint(-2**31, 2**31 - 1, (nbytes // 4,), dtype=torch.int32, device="cuda")
            for _ in range(n_sets)]
    sink = torch.zeros(4096, dtype=torch.int32, device="cuda")

    def timed(launch):
        torch.cuda.synchronize()            # the buffers were filled on the default stream
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            st = stream.cuda_stream
            for i in range(n_sets):
                launch(i, st)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for i in range(n_sets):
                    launch(i, st)
            g.replay()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            n = max(1, reps // n_sets)
            a.record(stream)
            for _ in range(n):
                g.replay()
            b.record(stream)
            torch.cuda.synchronize()
            return a.elapsed_time(b) * 1e3 / (n * n_sets)

    out = {"bytes": nbytes, "buffers": n_sets, "read": {}, "empty": {}}
    for blocks, threads, unroll, lds in ((256, 1024, 8, 0), (256, 768, 8, 0), (256, 768, 8, 147456),
                                         (512, 512, 8, 0), (1024, 256, 8, 0), (2048, 256, 4, 0),
                                         (4096, 256, 2, 0), (8192, 256, 1, 0)):
        def launch(i, st, b=blocks, t=threads, u=unroll, l=lds):
            rc = lib.probe_read(bufs[i].data_ptr(), nbytes, sink.data_ptr(), b, t, u, l, st)
            assert rc == 0, rc
        us = timed(launch)
        out["read"][f"{blocks}x{threads} unroll {unroll} lds {lds}"] = {
            "us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1)}
    for blocks, threads, lds in ((256, 768, 147456), (256, 768, 0), (256, 256, 0)):
        def launch(i, st, b=blocks, t=threads, l=lds):
            rc = lib.probe_empty(sink.data_ptr(), b, t, l, st)
            assert rc == 0, rc
        out["empty"][f"{blocks}x{threads} lds {lds}"] = {"us": round(timed(launch), 2)}
    return out


def decode_timeline(cfg: int = 2, rows=(1, 16)):
    """Clock stamps of the decode kernel's last launch over 18 rotating weight
    sets (a library built with QMM_TIMELINE=1 keeps them; `qmm_debug_stamps`
    copies them out): per wavefront role, the median over the workgroups of
    each stamp in microseconds after the launch's first wavefront starts.
    Returns {rows: {"compute first / second of a SIMD" | "loader": {stamp: us}}}."""
    import ctypes

    import numpy as np
    import torch

    from . import _lib, kernels, synth
    lib = _lib.load()
    if not hasattr(lib, "qmm_debug_stamps"):
        raise RuntimeError("this library keeps no clock stamps: build it with QMM_TIMELINE=1")
    compute = ["start", None, "activations in", "tile 0 published", "tile 0 computed", "tile 1 published",
               "tile 1 computed", "tile 2 published", "tile 2 computed", "tile 3 published", "tile 3 computed"]
    loader = ["start", "tile 0 requested", "tile 1 requested", "tile 0 landed", "tile 0 published",
              "tile 2 requested", "tile 1 landed", "tile 1 published", "tile 3 requested, tile 0 summed",
              "tile 2 landed", "tile 2 published", "tile 1 summed", "tile 3 landed", "tile 3 published",
              "tile 2 summed", "end"]
    out = {}
    for m in rows:
        wl = synth.make(cfg, M=m)
        sets = [synth.to_device(wl) for _ in range(18)]
        for x, w, s, b, _ in sets:
            kernels.quantized_matmul(x, w, s, b, group_size=64, bits=wl.bits)
        torch.cuda.synchronize()
        buf = np.zeros((256, 12, 16), dtype=np.uint64)
        rc = lib.qmm_debug_stamps(buf.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(buf.nbytes))
        if rc:
            raise RuntimeError(f"qmm_debug_stamps: {rc}")
        st = buf.astype(np.int64)
        us = (st - st[:, :, 0].min()) / 100.0               # the stamp clock runs at 100 MHz
        med = np.median(us, axis=0)
        rows_a_workgroup = -(-wl.N // 256)
        tiles = min(4, -(-rows_a_workgroup // 16))
        def pick(names, row, upto):
            return {n: round(float(row[i]), 2) for i, n in enumerate(names) if n and i < upto}
        out[f"M={m}"] = {
            "compute wavefronts 0-3 (first of their SIMD)": pick(compute, med[0:4].mean(axis=0), 3 + 2 * tiles),
            "compute wavefronts 4-7 (second of their SIMD)": pick(compute, med[4:8].mean(axis=0), 3 + 2 * tiles),
            "loaders": {**pick(loader, med[8:12].mean(axis=0), 3 + 3 * tiles), "end": round(float(med[8:12, 15].mean()), 2)},
        }
    return out


def main(argv):
    path = argv[1]
    total = sum(r[7] for r in kernel_stats(path)) or 1
    print("%-64s %9s %6s %7s %11s %11s %11s %6s" % ("kernel", "grid", "block", "calls", "avg_ns",
                                                      "min_ns", "max_ns", "time%"))
    for r in kernel_stats(path):
        print("%-64s %9d %6d %7d %11.0f %11d %11d %6.1f" % (_short(r[0]), r[1], r[2], r[3], r[4], r[5],
                                                             r[6], 100.0 * r[7] / total))
    cs = counter_stats(path)
    if cs:
        print()
        print("%-64s %-28s %16s %6s" % ("kernel", "counter", "mean/dispatch", "n"))
        for k, c, v, n in cs:
            print("%-64s %-28s %16.1f %6d" % (_short(k), c, v, n))


if __name__ == "__main__":
    main(sys.argv)
