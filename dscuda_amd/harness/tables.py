"""From timing samples to the files of a report.

The shape of the output is the reference's, because its tables are what these are laid beside
(``benchmarks/common.py:114-149``): one row per operation and reference backend with the columns

    size | dtype | operation | custom us | reference (<name>) us | reference %

where both times are medians over the trials and ``reference %`` = 100 * reference time / custom time (above 100 the
custom kernel is the faster one); per family the files ``<family>.csv``, ``<family>.md`` and ``<family>_samples.json``.
The samples file also carries, per operation, whatever facts the workload states about itself (flops or bytes), so
rates can be derived from it later.  Pure Python: nothing here needs a GPU.
"""

from __future__ import annotations

import csv
import json
import statistics
from dataclasses import asdict, dataclass
from pathlib import Path

CSV_FIELDS = ("size", "dtype", "operation", "custom_us", "reference", "reference_us", "reference_pct")
TIMING_NOTE = "HIP graph replay; warm-up and preparation excluded; median microseconds."


@dataclass(frozen=True)
class Row:
    size: str
    dtype: str
    operation: str
    custom_us: float | None
    reference: str
    reference_us: float | None
    reference_pct: float | None


def summarise(size: str, dtype: str, operation: str, samples: dict) -> list[Row]:
    """One row per backend other than ``custom``; a single row with reference ``none`` when there is no other."""
    custom = statistics.median(samples["custom"]) if samples.get("custom") else None
    rows = []
    for name, values in samples.items():
        if name == "custom" or not values:
            continue
        middle = statistics.median(values)
        rows.append(Row(size, dtype, operation, custom, name, middle, 100.0 * middle / custom if custom else None))
    return rows or [Row(size, dtype, operation, custom, "none", None, None)]


def _number(value, digits: int) -> str:
    return "—" if value is None else format(value, f".{digits}f")


def _table(reference: str, rows: list[Row]) -> str:
    grid = [["size", "dtype", "operation", "custom us", f"reference ({reference}) us", "reference %"]]
    grid += [[row.size, row.dtype, row.operation, _number(row.custom_us, 2), _number(row.reference_us, 2),
              _number(row.reference_pct, 1)] for row in rows]
    widths = [max(map(len, column)) for column in zip(*grid)]
    grid.insert(1, ["-" * width for width in widths])
    return "\n".join("| " + " | ".join(cell.ljust(width) for cell, width in zip(cells, widths)) + " |" for cells in grid)


def markdown(rows: list[Row]) -> str:
    """One table per reference backend, in order of first appearance."""
    by_reference: dict[str, list[Row]] = {}
    for row in rows:
        by_reference.setdefault(row.reference, []).append(row)
    return "\n\n".join(_table(reference, members) for reference, members in by_reference.items()) + "\n"


def write(directory, family: str, rows: list[Row], samples: list[dict], environment: dict) -> str:
    """Writes the three files of `family` below `directory` and returns the Markdown text."""
    if not rows:
        raise ValueError("no rows to report")
    target = Path(directory)
    target.mkdir(parents=True, exist_ok=True)
    with (target / f"{family}.csv").open("w", newline="") as handle:
        writer = csv.writer(handle)
        writer.writerow(CSV_FIELDS)
        for row in rows:
            record = asdict(row)
            writer.writerow(["" if record[name] is None else record[name] for name in CSV_FIELDS])
    text = markdown(rows)
    (target / f"{family}.md").write_text(text)
    document = dict(environment)
    document["timing"] = TIMING_NOTE
    document["samples"] = samples
    (target / f"{family}_samples.json").write_text(json.dumps(document, indent=2) + "\n")
    return text
