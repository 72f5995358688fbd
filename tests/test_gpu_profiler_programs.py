"""GPU run of the standalone profiler programs: each checks its own results against the closed form of its
inputs and exits non-zero on a mismatch."""

import json
import subprocess
from pathlib import Path

import pytest

BUILD = Path(__file__).resolve().parents[1] / "build"

CASES = [
    ("benchmark_mla", (1, 128, 8)),
    ("benchmark_mla", (2, 65, 3)),
    ("benchmark_mla", (1, 4096, 128)),          # the size the benchmark quotes: the cuts the library picks by itself there
    ("benchmark_mla_decode", (2, 1024, 16)),
    ("benchmark_mla_decode", (3, 129, 128, 512, 64, 4)),
    ("benchmark_mla_prefill", (1, 512, 4, 192, 128, "--constant", "--operation", "both")),
    ("benchmark_mla_prefill", (1, 1024, 8, 192, 128, "--operation", "both")),
    ("benchmark_flash_attention", (2, 256, 8, 128)),
    ("benchmark_flash_attention", (1, 512, 8, 64)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("program,arguments", CASES)
def test_program_checks_its_closed_forms(program, arguments):
    result = subprocess.run([str(BUILD / program), *map(str, arguments)], capture_output=True, text=True, timeout=120)
    assert result.returncode == 0, result.stderr + result.stdout
    assert "check " in result.stdout


@pytest.mark.gpu
def test_timing_line_parses():
    result = subprocess.run([str(BUILD / "benchmark_flash_attention"), "1", "512", "8", "64", "forward", "--timing",
                             "--warmup", "3", "--iterations", "5", "--trials", "3"],
                            capture_output=True, text=True, timeout=120)
    assert result.returncode == 0, result.stderr
    line = next(text for text in result.stdout.splitlines() if text.startswith("DSCUDA_TIMING "))
    record = json.loads(line[len("DSCUDA_TIMING "):])
    assert record["operation"] == "forward" and record["trials"] == 3
    assert 0.0 < record["minimum_ms"] <= record["median_ms"] <= record["maximum_ms"]
