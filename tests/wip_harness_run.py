"""GPU run of the runtime-table entry point.  Not collected by pytest under this name: its GPU path has not
been executed yet; run it by naming the file, and rename it to test_*.py once it has passed on a GPU."""

import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["flash_attention", "mla", "mla_prefill"])
def test_quick_suite_reports(family, tmp_path):
    result = subprocess.run([sys.executable, "-m", "dscuda_amd.harness.run", family, "--suite", "quick", "--warmup-ms", "50",
                             "--trials", "3", "--output", str(tmp_path)], capture_output=True, text=True, cwd=ROOT,
                            timeout=600)
    assert result.returncode == 0, result.stderr[-3000:]
    text = (tmp_path / f"{family}.md").read_text()
    assert "custom us" in text and "reference (PyTorch) us" in text
    assert (tmp_path / f"{family}.csv").is_file() and (tmp_path / f"{family}_samples.json").is_file()
