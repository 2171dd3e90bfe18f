#!/usr/bin/env python3
"""Text summaries of a rocprofv3 output directory (rocpd sqlite format), printed to stdout.

  python3 rust-autograd_amd/rocpd_summary.py trace DIR [--warmup W --steps K]
      per-kernel dispatch durations (microseconds) of a `--kernel-trace` run: count, min, median, mean and
      time per step.  With --warmup/--steps, a kernel launched a whole number of times per step has its
      warm-up dispatches dropped (the first W/(W+K) of them, in start order); other kernels list all dispatches.

  python3 rust-autograd_amd/rocpd_summary.py counters DIR
      per-kernel, per-counter average / min / max over dispatches of a `--pmc` run.

The tables under profiles/ are the output of this script over the commands each file names.
"""
import argparse
import collections
import glob
import re
import sqlite3
import statistics
import sys


def database(directory):
    found = sorted(glob.glob(f"{directory}/**/*.db", recursive=True))
    if not found:
        sys.exit(f"no rocpd database under {directory}")
    return sqlite3.connect(found[-1])


def short(name):
    """Kernel name without its argument list and return type."""
    return re.sub(r"\(.*", "", name).replace("void ", "")[:110]


def column(con, view, *candidates):
    cols = [r[1] for r in con.execute(f"pragma table_info({view})")]
    for c in candidates:
        if c in cols:
            return c
    sys.exit(f"view {view} has none of {candidates}: {cols}")


def trace(directory, warmup, steps):
    con = database(directory)
    name = column(con, "kernels", "name", "kernel_name")
    per = collections.defaultdict(list)
    for n, s, e in con.execute(f"select {name}, start, end from kernels order by start"):
        per[short(n)].append((e - s) / 1e3)
    lines = []
    for n, ds in per.items():
        total = warmup + steps
        if steps and len(ds) % total == 0:
            k = len(ds) // total
            timed, note = ds[warmup * k:], f"{k}/step, {warmup * k} warm-up dispatches dropped"
        else:
            timed, note = ds, "all dispatches"
        per_step = f"{sum(timed) / steps:11.2f}" if steps else f"{'-':>11s}"
        lines.append((sum(timed), f"{len(timed):5d} {min(timed):10.2f} {statistics.median(timed):10.2f} "
                                  f"{statistics.mean(timed):10.2f} {per_step}  {n}  ({note})"))
    print("    n     min_us  median_us    mean_us us_per_step  kernel")
    for _, line in sorted(lines, reverse=True):
        print(line)


def counters(directory):
    con = database(directory)
    views = [r[0] for r in con.execute("select name from sqlite_master where type in ('table','view')")
             if r[0].startswith("counters_collection")]
    if not views:
        sys.exit("no counters_collection view: not a --pmc run")
    view = views[0]
    kname = column(con, view, "kernel_name", "name")
    acc = collections.defaultdict(list)
    for n, c, v in con.execute(f"select {kname}, counter_name, value from {view}"):
        acc[(c, short(n))].append(v)
    for (c, n), vals in sorted(acc.items()):
        print(f"{c:26s} n={len(vals):3d} avg={sum(vals) / len(vals):16.1f} min={min(vals):16.1f} max={max(vals):16.1f}  {n}")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("what", choices=("trace", "counters"))
    ap.add_argument("directory")
    ap.add_argument("--warmup", type=int, default=0)
    ap.add_argument("--steps", type=int, default=0)
    a = ap.parse_args()
    if a.what == "trace":
        trace(a.directory, a.warmup, a.steps)
    else:
        counters(a.directory)


if __name__ == "__main__":
    main()
