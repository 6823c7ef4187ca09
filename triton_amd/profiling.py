"""Turn a rocprofv3 output database (the default `*_results.db` rocpd SQLite file) into a short text
summary: per-kernel call counts and average durations (`--kernel-trace --stats` runs) and per-kernel
counter values averaged per dispatch (`--pmc` runs).

    python -m triton_amd.profiling /tmp/prof/attn_results.db [--filter trn::] [--calib-bytes N] [--bench-json FILE]

Durations are given three ways: the plain average over every dispatch, the median, and the mean over the
dispatches that start later than --settle seconds (default 0.25) after the first dispatch of the trace.  The
plain average includes the cold call, the warm-ups and the first tens of milliseconds of a burst, during
which the board's clocks are still rising; the other two are the steady state that `bench.py` times.  With
--bench-json FILE (the JSON line `bench.py` printed in the profiled run) the header repeats that line's
ms_per_step and kernel_ms, so that the trace and the bench of one run on one board can be read side by side.

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


def kernel_stats(con, settle_s: float = 0.25):
    """(name, calls, total ns, average ns, median ns, steady-state mean ns, steady-state calls) per kernel from the
    dispatch trace; steady state = dispatches starting more than settle_s after the trace's first dispatch."""
    try:
        rows = list(con.execute("select name, start, end from kernels order by start"))
    except sqlite3.Error:
        return []
    if not rows:
        return []
    t0 = rows[0][1]
    per = collections.defaultdict(list)
    for name, start, end in rows:
        per[name].append((start, end - start))
    out = []
    for name, ds in per.items():
        durs = sorted(d for _, d in ds)
        steady = [d for st, d in ds if st - t0 > settle_s * 1e9]
        total = sum(durs)
        out.append((name, len(durs), total, total / len(durs), durs[len(durs) // 2],
                    sum(steady) / len(steady) if steady else float("nan"), len(steady)))
    out.sort(key=lambda r: -r[2])
    return out


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
    ap.add_argument("--settle", type=float, default=0.25, help="seconds after the first dispatch that count as warm-up")
    ap.add_argument("--bench-json", default="", help="file holding the JSON line bench.py printed in the profiled run")
    a = ap.parse_args()
    if a.bench_json:
        import json
        with open(a.bench_json) as f:
            lines = [ln for ln in f.read().splitlines() if ln.startswith("{")]
        if lines:
            b = json.loads(lines[-1])
            r = b.get("roofline", {})
            print(f"bench.py line of this run: ms_per_step {b.get('ms_per_step')}  roofline.kernel_ms {r.get('kernel_ms')}  "
                  f"roofline.achieved {r.get('achieved')} {r.get('unit')}  frac {r.get('frac')}  kernel {r.get('kernel')}")
    con = sqlite3.connect(a.db)
    stats = [r for r in kernel_stats(con, a.settle) if a.filter in r[0]]
    if stats:
        print(f"{'kernel':72s} {'calls':>6s} {'avg_us':>10s} {'median_us':>10s} {'steady_us':>10s} {'(calls)':>8s} {'total_us':>11s}")
        for name, calls, total, avg, med, steady, nst in stats:
            print(f"{short(name):72s} {calls:6d} {avg / 1e3:10.2f} {med / 1e3:10.2f} {steady / 1e3:10.2f} {nst:8d} {total / 1e3:11.1f}")
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
