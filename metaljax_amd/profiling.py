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
