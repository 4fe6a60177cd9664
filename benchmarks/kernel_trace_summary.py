#!/usr/bin/env python3
"""Kernel time by name from a ``rocprofv3 --kernel-trace --output-format csv`` output folder, as a markdown table:

    python benchmarks/kernel_trace_summary.py DIR [--title TEXT] [--rows N] > kernels.md

Reads every ``*kernel_trace.csv`` under DIR (columns ``Kernel_Name``, ``Start_Timestamp``, ``End_Timestamp`` in
ns), groups the launches by kernel name with the template arguments kept and the parameter list dropped, and prints
total / share / calls / average / minimum / maximum per name, largest total first.
"""
from __future__ import annotations

import argparse
import csv
import glob
import os
import re
import sys


def short(name: str) -> str:
    name = re.sub(r"^void\s+", "", name)
    name = re.sub(r"\(anonymous namespace\)::", "", name)
    depth, out = 0, []
    for ch in name:                      # drop the parameter list: everything from the first '(' outside <...>
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            break
        out.append(ch)
    s = "".join(out).strip()
    s = s.replace("unsigned short", "bf16").replace("(bool)1", "true").replace("(bool)0", "false")
    s = re.sub(r"\((?:int|long|bool)\)", "", s)
    return s[:110]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("dir")
    ap.add_argument("--title", default="kernel time by name")
    ap.add_argument("--rows", type=int, default=50)
    a = ap.parse_args(argv)
    files = glob.glob(os.path.join(a.dir, "**", "*kernel_trace.csv"), recursive=True)
    if not files:
        print(f"no *kernel_trace.csv under {a.dir}", file=sys.stderr)
        return 1
    stats: dict = {}
    for f in files:
        with open(f, newline="") as fh:
            for row in csv.DictReader(fh):
                us = (int(row["End_Timestamp"]) - int(row["Start_Timestamp"])) / 1e3
                s = stats.setdefault(short(row["Kernel_Name"]), [0.0, 0, float("inf"), 0.0])
                s[0] += us
                s[1] += 1
                s[2] = min(s[2], us)
                s[3] = max(s[3], us)
    total = sum(s[0] for s in stats.values())
    print(f"## {a.title}\n")
    print("| total us | % | calls | avg us | min us | max us | kernel |")
    print("|---:|---:|---:|---:|---:|---:|---|")
    for name, s in sorted(stats.items(), key=lambda kv: -kv[1][0])[: a.rows]:
        print(f"| {s[0]:.0f} | {100 * s[0] / total:.1f} | {s[1]} | {s[0] / s[1]:.1f} | {s[2]:.1f} | {s[3]:.1f} | `{name}` |")
    return 0


if __name__ == "__main__":
    sys.exit(main())
