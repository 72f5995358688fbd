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


def test_closed_forms_checked_by_benchmark_mla_prefill_hold_for_the_oracle():
    """The constant inputs of `benchmark_mla_prefill --constant` and the closed forms the program compares the
    kernels with (its header comment), evaluated with the fp32 oracle on a small shape."""
    import math
    import torch
    from oracle import attention_oracle as oracle
    batch, seq, heads, d_qk, d_v = 1, 40, 2, 192, 128
    scale = 1.0 / math.sqrt(d_qk)
    q = torch.full((batch, seq, heads, d_qk), 0.125).bfloat16()
    k = torch.full((batch, seq, heads, d_qk), 0.25).bfloat16()
    v = torch.full((batch, seq, heads, d_v), 0.5).bfloat16()
    dout = torch.full((batch, seq, heads, d_v), 0.015625).bfloat16()
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    score = d_qk * 0.125 * 0.25 * scale
    assert torch.allclose(out.float(), torch.full_like(out.float(), 0.5), atol=1e-6)
    expected_lse = score + torch.log(torch.arange(1, seq + 1, dtype=torch.float32))
    assert torch.allclose(lse, expected_lse.expand(batch, heads, seq), atol=1e-5)
    dq, dk, dv = oracle.attention_backward(dout, out.bfloat16(), lse, q, k, v, scale)
    assert dq.float().abs().max() < 1e-6 and dk.float().abs().max() < 1e-6
    harmonic = torch.cumsum(1.0 / torch.arange(1, seq + 1, dtype=torch.float64), 0)
    harmonic = torch.cat((torch.zeros(1, dtype=torch.float64), harmonic))          # Harm(0..S)
    expected_dv = 0.015625 * (harmonic[seq] - harmonic[:seq])                       # per key
    assert torch.allclose(dv.float()[0, :, 0, 0].double(), expected_dv, atol=1e-6)
    assert torch.allclose(dv.float(), dv.float()[:, :, :1, :1].expand_as(dv), atol=1e-7)
