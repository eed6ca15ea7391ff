"""Per-kernel sums of one step out of a ``rocprofv3 --kernel-trace`` run.

    rocprofv3 --kernel-trace --output-format csv -d OUT -- python3 bench.py --steps 16 --warmup 4 --no-points
    python -m xyntetik_runner_amd.profile_summary OUT --marker k_sample            # the last decode step
    python -m xyntetik_runner_amd.profile_summary OUT --marker k_embedding --grid 524288   # a prompt step of 2,048 rows

A step is what lies between two dispatches of a marker kernel (the pick ends a decode step, the
embedding begins a prompt step).  ``--grid N`` takes only spans whose marker dispatch has a grid of
at least N threads (the embedding of a 2,048-row step, 256 threads a row, among those of decode
steps); ``--index``
counts spans from the end (-1: the last).  The table is markdown, as the files under ``profiles/``
hold it.

    rocprofv3 --pmc SQ_CYCLES SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES --kernel-trace --output-format csv -d OUT -- python3 bench.py ...
    python -m xyntetik_runner_amd.profile_summary OUT --counters --kernel k_attn_cta --kernel k_gemm_tile

``--counters`` reads the counters of such a run instead: for every kernel whose name holds one of the
``--kernel`` strings (all kernels without), the dispatches (``--grid N``: those of at least N
threads), their mean time and the mean of every counter per dispatch.

The reference prints per-op timings of a decode step from inside its engine
(src/main.c:1435-1515 for its own bench); here the profiler's trace is the source.
"""
from __future__ import annotations

import argparse
import csv
import glob
import os
import re
import sys
from typing import Dict, List, Tuple


def read_trace(folder: str) -> List[Tuple[int, int, str, int]]:
    """(start ns, end ns, kernel name, grid size) of every dispatch, in order of start."""
    files = sorted(glob.glob(os.path.join(folder, "**", "*kernel_trace.csv"), recursive=True), key=os.path.getmtime)
    if not files:
        raise SystemExit(f"no *kernel_trace.csv under {folder}")
    rows = []
    with open(files[-1], newline="") as f:               # the newest, if the folder holds several runs
        for r in csv.DictReader(f):
            rows.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Kernel_Name"], int(r.get("Grid_Size_X") or 0)))
    rows.sort()
    return rows


def short_name(name: str) -> str:
    """``k_gemm_skinny<1, 1, 8, 8, true, true>(GemmArgs)`` -> ``k_gemm_skinny<1,1,8,8,true,true>``."""
    name = re.sub(r"\(.*\)$", "", name.split(" [clone")[0]).strip()
    if name.startswith("void "):
        name = name[5:]
    return name.replace(", ", ",")


def spans(rows, marker: str, min_grid: int) -> List[Tuple[int, int]]:
    """[first, last) row indices of the steps: from one marker dispatch to the next."""
    at = [i for i, r in enumerate(rows) if marker in r[2] and r[3] >= min_grid]
    every = [i for i, r in enumerate(rows) if marker in r[2]]
    out = []
    for i in at:
        later = [j for j in every if j > i]
        if later:
            out.append((i, later[0]))
    return out


def summarize(rows, first: int, last: int) -> str:
    step = rows[first:last]
    agg: Dict[str, List[int]] = {}
    for s, e, name, _ in step:
        a = agg.setdefault(short_name(name), [0, 0])
        a[0] += 1
        a[1] += e - s
    busy = sum(t for _, t in agg.values())
    span = step[-1][1] - step[0][0] if step else 0
    lines = [f"{len(step)} kernels, span {span / 1e3:,.0f} us, kernels busy {busy / 1e3:,.0f} us", "",
             "| time (us) | share | calls x mean (us) | kernel |", "|----------:|------:|-------------------|--------|"]
    for name, (n, t) in sorted(agg.items(), key=lambda kv: -kv[1][1]):
        lines.append(f"| {t / 1e3:,.1f} | {100.0 * t / max(busy, 1):.1f}% | {n} x {t / n / 1e3:.1f} | `{name}` |")
    return "\n".join(lines)


def read_counters(folder: str, min_grid: int = 0) -> Dict[str, Dict[str, List[float]]]:
    """kernel name -> counter name -> one value per dispatch (and "us": the dispatches' times)."""
    files = sorted(glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True), key=os.path.getmtime)
    if not files:
        raise SystemExit(f"no *counter_collection.csv under {folder}")
    out: Dict[str, Dict[str, List[float]]] = {}
    seen = set()
    with open(files[-1], newline="") as f:
        for r in csv.DictReader(f):
            if int(r.get("Grid_Size") or 0) < min_grid:
                continue
            k = out.setdefault(short_name(r["Kernel_Name"]), {})
            k.setdefault(r["Counter_Name"], []).append(float(r["Counter_Value"]))
            if r["Dispatch_Id"] not in seen:             # a dispatch has a row per counter, with the same times
                seen.add(r["Dispatch_Id"])
                k.setdefault("us", []).append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    return out


def counter_table(counters: Dict[str, Dict[str, List[float]]], kernels: List[str]) -> str:
    names = [n for n in counters if not kernels or any(k in n for k in kernels)]
    cols = sorted({c for n in names for c in counters[n] if c != "us"})
    lines = ["| kernel | dispatches | mean us | " + " | ".join(cols) + " |", "|--------|-----------:|--------:|" + "|".join("-" * (len(c) + 1) + ":" for c in cols) + "|"]
    for n in sorted(names, key=lambda n: -sum(counters[n].get("us", [0]))):
        c = counters[n]
        us = c.get("us", [0.0])
        cells = [f"{sum(c[x]) / len(c[x]):,.0f}" if x in c else "" for x in cols]
        lines.append(f"| `{n}` | {len(us)} | {sum(us) / len(us):,.1f} | " + " | ".join(cells) + " |")
    return "\n".join(lines)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="profile_summary", description=__doc__.split("\n\n")[0])
    ap.add_argument("folder", help="the -d folder of the rocprofv3 run")
    ap.add_argument("--marker", default="k_sample", help="part of the name of the kernel that separates steps")
    ap.add_argument("--grid", type=int, default=0, help="only spans whose marker dispatch has at least this many threads")
    ap.add_argument("--index", type=int, default=-1, help="which span, counted from the end (-1: the last)")
    ap.add_argument("--counters", action="store_true", help="the means of a --pmc run's counters per kernel instead of a step's times")
    ap.add_argument("--kernel", action="append", default=[], help="with --counters: only kernels whose name holds this (may be given again)")
    args = ap.parse_args(argv)
    if args.counters:
        print(counter_table(read_counters(args.folder, args.grid), args.kernel))
        return 0
    rows = read_trace(args.folder)
    found = spans(rows, args.marker, args.grid)
    if not found:
        names = sorted({short_name(r[2]) for r in rows})
        raise SystemExit(f"no two dispatches of a kernel named *{args.marker}* (grid >= {args.grid}); kernels seen: {names}")
    first, last = found[args.index]
    print(summarize(rows, first, last))
    return 0


if __name__ == "__main__":
    sys.exit(main())
