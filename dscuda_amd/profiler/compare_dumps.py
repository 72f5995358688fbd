"""Compares two raw fp32 dumps of one tensor written by different processes.

The standalone programs write their forward output as raw fp32 when given a file
name (``profiler_common.h: dump_as_float``); this is the checker for two such
files, the counterpart of the reference's ``scripts/compare_attention_dumps.py``:

    python -m dscuda_amd.profiler.compare_dumps A.bin B.bin BATCH SEQUENCE HEADS HEAD_SIZE [--tolerance T]

Prints max-abs and RMS difference and exits non-zero when max-abs exceeds the tolerance
or a file does not hold BATCH*SEQUENCE*HEADS*HEAD_SIZE floats.
"""

from __future__ import annotations

import argparse
import sys
from pathlib import Path

import numpy as np


def compare(left_path: Path, right_path: Path, elements: int, tolerance: float):
    sizes = [path.stat().st_size // 4 for path in (left_path, right_path)]
    if sizes != [elements, elements]:
        raise ValueError(f"expected {elements} floats per dump; got {sizes[0]} and {sizes[1]}")
    left = np.memmap(left_path, dtype=np.float32, mode="r")
    right = np.memmap(right_path, dtype=np.float32, mode="r")
    worst, squares = 0.0, 0.0
    step = 1 << 22
    for begin in range(0, elements, step):
        difference = left[begin:begin + step].astype(np.float64) - right[begin:begin + step]
        if not np.isfinite(difference).all():
            return float("inf"), float("inf"), False
        worst = max(worst, float(np.abs(difference).max()))
        squares += float((difference * difference).sum())
    rms = (squares / elements) ** 0.5
    return worst, rms, worst <= tolerance


def main(argv=None):
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("left", type=Path)
    parser.add_argument("right", type=Path)
    parser.add_argument("batch", type=int)
    parser.add_argument("sequence", type=int)
    parser.add_argument("heads", type=int)
    parser.add_argument("head_size", type=int)
    parser.add_argument("--tolerance", type=float, default=2.5e-2)
    args = parser.parse_args(argv)
    elements = args.batch * args.sequence * args.heads * args.head_size
    try:
        worst, rms, passed = compare(args.left, args.right, elements, args.tolerance)
    except ValueError as error:
        print(error, file=sys.stderr)
        return 2
    print(f"{'tensor':<10} {'max abs':>12} {'RMS':>12} {'result':>9}")
    print(f"{'output':<10} {worst:>12.4e} {rms:>12.4e} {('PASS' if passed else 'FAIL'):>9}")
    return 0 if passed else 1


if __name__ == "__main__":
    sys.exit(main())
