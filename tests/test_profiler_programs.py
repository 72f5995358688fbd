"""Host-only checks of the standalone profiler programs (dscuda_amd/profiler/*.cpp, linked into build/ by
`python -m dscuda_amd.build`): they exist, refuse bad arguments with a message and status 1, and fail
cleanly -- message on stderr, status 1 -- where no GPU is present.  What they compute is checked by the
programs themselves on a GPU (closed forms of their constant inputs)."""

import subprocess
from pathlib import Path

import pytest

BUILD = Path(__file__).resolve().parents[1] / "build"
PROGRAMS = ["benchmark_mla", "benchmark_mla_decode", "benchmark_mla_prefill", "benchmark_flash_attention"]


def run(program, *arguments):
    return subprocess.run([str(BUILD / program), *map(str, arguments)], capture_output=True, text=True, timeout=120)


@pytest.mark.parametrize("program", PROGRAMS)
def test_program_is_built(program):
    assert (BUILD / program).is_file(), f"{program} missing: run python -m dscuda_amd.build"


@pytest.mark.parametrize("program,arguments,message", [
    ("benchmark_mla", (0,), "batch must be a positive integer"),
    ("benchmark_mla_decode", (2, 1024, 16, 512, 64, 0), "splits must be a positive integer"),
    ("benchmark_mla_prefill", (1, 64, 2, 192, 128, "--operation", "sideways"), "--operation is forward, backward or both"),
    ("benchmark_mla_prefill", (1, 64, 2, 192, 128, "--bogus"), "unknown option --bogus"),
    ("benchmark_flash_attention", (1, 64, 2, 128, "backward"), "only forward is supported"),
    ("benchmark_flash_attention", (1, 64, 2, 128, "forward", "--timing", "--trials"), "--trials needs a value"),
])
def test_bad_arguments_are_refused_before_any_gpu_call(program, arguments, message):
    result = run(program, *arguments)
    assert result.returncode == 1
    assert message in result.stderr
    assert "HIP failure" not in result.stderr


@pytest.mark.parametrize("program,arguments", [
    ("benchmark_mla", (1, 64, 2)),
    ("benchmark_mla_decode", (1, 128, 4)),
    ("benchmark_mla_prefill", (1, 64, 2, 192, 128, "--constant")),
    ("benchmark_flash_attention", (1, 64, 2, 128)),
])
def test_valid_invocation_succeeds_or_reports_the_missing_gpu(program, arguments):
    result = run(program, *arguments)
    if result.returncode == 0:
        assert "workload:" in result.stdout
    else:
        assert result.returncode == 1
        assert "benchmark failed: HIP failure" in result.stderr
