"""GPU run of the runtime-table entry point (dscuda_amd/harness/run.py): the correctness mode on the reference
harness's test shapes, the timed quick suites with their three report files, the h100 decode suite without a
reference, and the profiler mode."""

import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
pytestmark = pytest.mark.gpu


def harness(*arguments, timeout=900):
    return subprocess.run([sys.executable, "-m", "dscuda_amd.harness.run", *map(str, arguments)], capture_output=True,
                          text=True, cwd=ROOT, timeout=timeout)


@pytest.mark.parametrize("family,checks", [("flash_attention", 4), ("mla", 10), ("mla_prefill", 4)])
def test_correctness_mode(family, checks):
    result = harness(family, "--test")
    assert result.returncode == 0, result.stderr[-3000:]
    assert f"{family}: {checks} correctness checks passed" in result.stdout


@pytest.mark.parametrize("family", ["flash_attention", "mla", "mla_prefill"])
def test_quick_suite_reports(family, tmp_path):
    result = harness(family, "--suite", "quick", "--warmup-ms", 50, "--trials", 3, "--output", tmp_path)
    assert result.returncode == 0, result.stderr[-3000:]
    text = (tmp_path / f"{family}.md").read_text()
    assert text == result.stdout
    assert "custom us" in text and "reference (PyTorch) us" in text
    assert (tmp_path / f"{family}.csv").is_file() and (tmp_path / f"{family}_samples.json").is_file()


def test_h100_decode_suite_without_a_reference(tmp_path):
    result = harness("mla", "--suite", "h100", "--reference", "none", "--warmup-ms", 50, "--trials", 3, "--output", tmp_path)
    assert result.returncode == 0, result.stderr[-3000:]
    lines = [line for line in result.stdout.splitlines() if line.startswith("| B=")]
    assert len(lines) == 4 and all("decode" in line for line in lines)
    assert "reference (none) us" in result.stdout


def test_profile_mode_announces_each_call():
    result = harness("mla", "--suite", "quick", "--operation", "decode", "--profile", "--backend", "custom")
    assert result.returncode == 0, result.stderr[-3000:]
    assert result.stdout.count("profile: ") == 1 and "/custom/decode" in result.stdout
