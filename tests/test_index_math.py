"""Builds tests/host/index_math_test.cpp with the host compiler and runs it: exhaustive checks of the integer
arithmetic the kernels take from dscuda_amd/csrc/index_math.h (LDS chunk permutations and their bank spread,
fast vs general tile-request offsets, dS block numbering, the forward work order, the decode range split)."""

import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def test_index_math_host_checks(tmp_path):
    compiler = shutil.which("g++") or shutil.which("c++")
    if compiler is None:
        pytest.skip("no host C++ compiler")
    binary = tmp_path / "index_math_test"
    build = subprocess.run([compiler, "-std=c++17", "-O1", "-Wall", "-Werror", f"-I{ROOT / 'dscuda_amd' / 'csrc'}",
                            str(ROOT / "tests" / "host" / "index_math_test.cpp"), "-o", str(binary)],
                           capture_output=True, text=True, timeout=300)
    assert build.returncode == 0, build.stderr
    result = subprocess.run([str(binary)], capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stdout[-4000:]
    assert "all checks passed" in result.stdout
