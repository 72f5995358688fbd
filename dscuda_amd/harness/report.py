"""Timing records and the six-column runtime table of the reference's harness
(``benchmarks/common.py:42-61,114-149``): size | dtype | operation | custom us |
reference (<name>) us | reference %.  Pure Python, no GPU: ``run.py`` feeds it
the per-trial samples it measures.

``reference %`` keeps the reference's meaning: 100 * reference time / custom
time, i.e. above 100 the custom kernel is the faster one.
"""

from __future__ import annotations

import csv
import json
import math
import statistics
from dataclasses import dataclass, field
from pathlib import Path

HEADERS = ("size", "dtype", "operation", "custom us", "reference ({}) us", "reference %")


@dataclass
class Operation:
    """One timed operation: its label columns, the backends (name -> zero-argument
    callable returning the outputs; "custom" is this library) and a checker that
    raises AssertionError when outputs are off (None: nothing to compare with)."""
    size: str
    dtype: str
    name: str
    functions: dict
    check: object = None
    notes: dict = field(default_factory=dict)


def repeats_for(sample_ms: float, per_replay_ms: float) -> int:
    """Replays per timing sample so that one sample lasts about `sample_ms`
    (``benchmarks/common.py:97-98``)."""
    return max(1, math.ceil(sample_ms / max(per_replay_ms, 1e-6)))


def trial_order(names, trial: int):
    """Backends alternate direction from trial to trial so that none always runs
    on a warmer chip than the other (``benchmarks/common.py:101-103``)."""
    names = list(names)
    return names if trial % 2 == 0 else names[::-1]


def record(operation: Operation, samples: dict) -> list[dict]:
    """One row per reference backend; a custom-only operation yields one row with
    an empty reference."""
    custom = statistics.median(samples["custom"]) if samples.get("custom") else None
    rows = [dict(size=operation.size, dtype=operation.dtype, operation=operation.name, custom_us=custom,
                 reference=name, reference_us=statistics.median(values),
                 reference_pct=100.0 * statistics.median(values) / custom if custom else None)
            for name, values in samples.items() if name != "custom" and values]
    if not rows:
        rows.append(dict(size=operation.size, dtype=operation.dtype, operation=operation.name, custom_us=custom,
                         reference="none", reference_us=None, reference_pct=None))
    return rows


def _cell(value, digits):
    return "—" if value is None else f"{value:.{digits}f}"


def render_tables(rows: list[dict]) -> str:
    """Markdown: one table per reference backend, columns padded to a common width."""
    tables = []
    for reference in dict.fromkeys(row["reference"] for row in rows):
        selected = [row for row in rows if row["reference"] == reference]
        headers = [text.format(reference) for text in HEADERS]
        cells = [[row["size"], row["dtype"], row["operation"], _cell(row["custom_us"], 2),
                  _cell(row["reference_us"], 2), _cell(row["reference_pct"], 1)] for row in selected]
        widths = [max(len(line[column]) for line in [headers, *cells]) for column in range(len(headers))]

        def line(values):
            return "| " + " | ".join(value.ljust(width) for value, width in zip(values, widths)) + " |"

        tables.append("\n".join([line(headers), line(["-" * width for width in widths]), *map(line, cells)]))
    return "\n\n".join(tables) + "\n"


def save_report(directory, family: str, rows: list[dict], samples: list[dict], environment: dict) -> str:
    """Writes <family>.csv, <family>.md and <family>_samples.json below `directory`
    (the reference writes the same three files, ``benchmarks/common.py:133-142``)
    and returns the Markdown."""
    if not rows:
        raise ValueError("no rows to report")
    destination = Path(directory)
    destination.mkdir(parents=True, exist_ok=True)
    with (destination / f"{family}.csv").open("w", newline="") as handle:
        writer = csv.DictWriter(handle, fieldnames=list(rows[0]))
        writer.writeheader()
        writer.writerows(rows)
    report = render_tables(rows)
    (destination / f"{family}.md").write_text(report)
    (destination / f"{family}_samples.json").write_text(json.dumps({
        **environment,
        "timing": "HIP graph replay; warm-up and preparation excluded; median microseconds.",
        "samples": samples}, indent=2) + "\n")
    return report
