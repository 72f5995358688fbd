"""Condenses ``rocprofv3 --output-format csv`` output into the few lines worth
keeping: per-kernel call count and average duration from a ``--kernel-trace
--stats`` run, per-kernel counter averages from a ``--pmc`` run.

    python3 dscuda_amd/harness/profile_summary.py --command "<what was run>" DIR [DIR ...]

Every ``*_kernel_stats.csv`` and ``*_counter_collection.csv`` below each DIR is
read; output is plain text on stdout.
"""

from __future__ import annotations

import argparse
import collections
import csv
from pathlib import Path


def short_name(name: str) -> str:
    name = name.replace("void ", "").replace("(anonymous namespace)::", "").replace("dscuda::", "")
    cut = name.find("(")
    return name if cut < 0 else name[:cut]


def wanted(name: str, patterns: list[str]) -> bool:
    return not patterns or any(pattern in name for pattern in patterns)


def kernel_stats(path: Path, patterns: list[str]) -> list[str]:
    lines = [f"{'kernel':78s} {'calls':>6s} {'avg us':>10s} {'min us':>10s} {'max us':>10s} {'%':>6s}"]
    with open(path, newline="") as handle:
        for row in csv.DictReader(handle):
            if not wanted(row["Name"], patterns):
                continue
            lines.append(f"{short_name(row['Name'])[:78]:78s} {int(row['Calls']):6d} "
                         f"{float(row['AverageNs']) / 1e3:10.1f} {float(row['MinNs']) / 1e3:10.1f} "
                         f"{float(row['MaxNs']) / 1e3:10.1f} {float(row['Percentage']):6.2f}")
    return lines


def mean(values) -> float:
    values = list(values)
    return sum(values) / len(values)


def counter_averages(path: Path, patterns: list[str], xcds: int = 8) -> list[str]:
    """Counter means per kernel.  Where the file carries dispatch timestamps, also
    the dispatch duration of the first launches and of the second half of them
    (the chip's clock takes some tens of launches to settle), and, if
    GRBM_GUI_ACTIVE was collected (it is summed over the `xcds` dies), the clock
    those cycles imply."""
    table = collections.defaultdict(lambda: collections.defaultdict(list))
    spans = collections.defaultdict(lambda: collections.defaultdict(list))
    with open(path, newline="") as handle:
        for row in csv.DictReader(handle):
            if not wanted(row["Kernel_Name"], patterns):
                continue
            kernel = short_name(row["Kernel_Name"])
            table[kernel][row["Counter_Name"]].append(float(row["Counter_Value"]))
            if row.get("Start_Timestamp") and row.get("End_Timestamp"):
                spans[kernel][row["Counter_Name"]].append(int(row["End_Timestamp"]) - int(row["Start_Timestamp"]))
    lines = []
    for kernel, counters in table.items():
        lines.append(kernel[:100])
        for counter, values in counters.items():
            lines.append(f"    {counter:32s} {mean(values):18.1f}   (mean of {len(values)} dispatches)")
        durations = next(iter(spans[kernel].values()), [])
        if len(durations) >= 8:
            head, tail = durations[:5], durations[len(durations) // 2:]
            lines.append(f"    dispatch duration: first {len(head)} launches {mean(head) / 1e3:.1f} us, "
                         f"second half ({len(tail)} launches) {mean(tail) / 1e3:.1f} us")
            cycles = counters.get("GRBM_GUI_ACTIVE")
            if cycles and len(cycles) == len(durations):
                half = len(cycles) // 2
                lines.append(f"    clock from GRBM_GUI_ACTIVE / {xcds} dies: first launches "
                             f"{mean(cycles[:5]) / xcds / mean(head):.2f} GHz, second half "
                             f"{mean(cycles[half:]) / xcds / mean(tail):.2f} GHz")
        elif durations:
            lines.append(f"    dispatch duration: {mean(durations) / 1e3:.1f} us (mean of {len(durations)})")
    return lines


def main():
    parser = argparse.ArgumentParser(description=__doc__)
    parser.add_argument("--command", required=True, help="the profiled command line, recorded in the summary")
    parser.add_argument("--only", action="append", default=[],
                        help="keep kernels whose name contains this text (repeatable; default: dscuda and copy kernels)")
    parser.add_argument("directories", nargs="+")
    args = parser.parse_args()
    patterns = args.only or ["dscuda", "copyBuffer"]
    print(f"command: {args.command}")
    for directory in args.directories:
        for path in sorted(Path(directory).rglob("*_kernel_stats.csv")):
            print(f"\n[kernel trace] {path.name}")
            print("\n".join(kernel_stats(path, patterns)))
        for path in sorted(Path(directory).rglob("*_counter_collection.csv")):
            print(f"\n[counters] {path.name}")
            print("\n".join(counter_averages(path, patterns)))


if __name__ == "__main__":
    main()
