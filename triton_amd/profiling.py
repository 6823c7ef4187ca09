"""Turn a rocprofv3 output database (the default `*_results.db` rocpd SQLite file) into a short text
summary: per-kernel call counts and average durations (`--kernel-trace --stats` runs) and per-kernel
counter values averaged per dispatch (`--pmc` runs).

    python -m triton_amd.profiling /tmp/prof/attn_results.db [--filter trn::] [--calib-bytes N]

With --calib-bytes N the FETCH_SIZE / WRITE_SIZE readings (KiB per dispatch) of every kernel are also
shown scaled by what the library's calibration copy kernel read for its known N bytes.
"""
from __future__ import annotations

import argparse
import collections
import sqlite3


def short(name: str) -> str:
    name = name.split("(")[0]
    return name[-72:]


def kernel_stats(con):
    """(name, calls, total ns, average ns) per kernel from the dispatch trace."""
    try:
        rows = list(con.execute("select name, count(*), sum(end - start), avg(end - start) from kernels "
                                "group by name order by sum(end - start) desc"))
    except sqlite3.Error:
        return []
    return rows


def counters(con):
    """Per kernel: counter sums, dispatch ids and summed durations; plus per-(kernel, grid size) sums so that
    the calibration copy of one particular size can be singled out."""
    agg = collections.defaultdict(lambda: collections.defaultdict(float))
    disp = collections.defaultdict(set)
    dur = collections.defaultdict(float)
    bygrid = collections.defaultdict(lambda: collections.defaultdict(float))
    gdisp = collections.defaultdict(set)
    try:
        cur = con.execute("select kernel_name, dispatch_id, counter_name, value, duration, grid_size from counters_collection")
    except sqlite3.Error:
        return {}, {}, {}, {}, {}
    seen = set()
    for name, d, cname, val, du, grid in cur:
        agg[name][cname] += val
        disp[name].add(d)
        bygrid[(name, grid)][cname] += val
        gdisp[(name, grid)].add(d)
        if (name, d) not in seen:
            seen.add((name, d)); dur[name] += du
    return agg, disp, dur, bygrid, gdisp


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("db")
    ap.add_argument("--filter", default="trn", help="only kernels whose name contains this (default: this library's)")
    ap.add_argument("--calib-bytes", type=int, default=0)
    a = ap.parse_args()
    con = sqlite3.connect(a.db)
    stats = [r for r in kernel_stats(con) if a.filter in r[0]]
    if stats:
        print(f"{'kernel':72s} {'calls':>6s} {'avg_us':>10s} {'total_us':>11s}")
        for name, calls, total, avg in stats:
            print(f"{short(name):72s} {calls:6d} {avg / 1e3:10.2f} {total / 1e3:11.1f}")
    agg, disp, dur, bygrid, gdisp = counters(con)
    calib = {}
    for (name, grid), vals in bygrid.items():       # the copy launched on exactly --calib-bytes (16 bytes per work-item)
        if "calibration_copy" in name and a.calib_bytes and grid == a.calib_bytes // 16:
            calib = {c: v / len(gdisp[(name, grid)]) for c, v in vals.items()}
            print(f"\ncalibration copy of {a.calib_bytes} bytes: " + ", ".join(f"{c}={v:.1f}" for c, v in sorted(calib.items()))
                  + f"  ({len(gdisp[(name, grid)])} dispatches)")
    for name in agg:
        if a.filter not in name:
            continue
        n = len(disp[name])
        print(f"\n{short(name)}  dispatches={n} avg_us={dur[name] / n / 1e3:.2f}")
        for c, v in sorted(agg[name].items()):
            line = f"    {c:32s} {v / n:18.1f} per dispatch"
            if a.calib_bytes and c in calib and calib[c] > 0 and c in ("FETCH_SIZE", "WRITE_SIZE"):
                line += f"   -> {v / n / calib[c] * a.calib_bytes:16.0f} bytes (scaled by the {a.calib_bytes}-byte copy)"
            print(line)


if __name__ == "__main__":
    main()
