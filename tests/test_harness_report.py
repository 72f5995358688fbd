"""Host-only checks of the runtime-table code (dscuda_amd/harness/report.py) and of the argument handling of
the harness entry point (dscuda_amd/harness/run.py): medians, the reference-percent convention, table layout
and the three report files, on numbers whose answers can be read off."""

import csv
import json
import subprocess
import sys
from pathlib import Path

import pytest

from dscuda_amd.harness import report

ROOT = Path(__file__).resolve().parents[1]


def operation(name="forward", notes=None):
    return report.Operation("B=1,T=512", "bf16", name, {"custom": None, "PyTorch": None}, None, notes or {})


def test_repeats_cover_the_sample_window():
    assert report.repeats_for(20, 0.5) == 40
    assert report.repeats_for(20, 0.3) == 67        # ceil
    assert report.repeats_for(20, 100.0) == 1       # never zero
    assert report.repeats_for(20, 0.0) >= 1         # a zero measurement does not divide by zero


def test_trial_order_alternates():
    assert report.trial_order(["custom", "PyTorch"], 0) == ["custom", "PyTorch"]
    assert report.trial_order(["custom", "PyTorch"], 1) == ["PyTorch", "custom"]


def test_record_uses_medians_and_reference_percent():
    rows = report.record(operation(), {"custom": [10.0, 30.0, 20.0], "PyTorch": [100.0, 50.0, 60.0]})
    assert len(rows) == 1
    row = rows[0]
    assert row["custom_us"] == 20.0 and row["reference_us"] == 60.0 and row["reference"] == "PyTorch"
    assert row["reference_pct"] == pytest.approx(300.0)    # the reference takes three times as long


def test_record_without_a_reference_keeps_the_custom_time():
    rows = report.record(operation(), {"custom": [4.0, 6.0]})
    assert rows == [dict(size="B=1,T=512", dtype="bf16", operation="forward", custom_us=5.0, reference="none",
                         reference_us=None, reference_pct=None)]


def test_record_with_two_references_gives_two_rows():
    rows = report.record(operation(), {"custom": [2.0], "PyTorch": [8.0], "Other": [1.0]})
    assert [(row["reference"], row["reference_pct"]) for row in rows] == [("PyTorch", 400.0), ("Other", 50.0)]


def test_tables_are_grouped_by_reference_and_aligned():
    rows = report.record(operation(), {"custom": [2.0], "PyTorch": [8.0], "Other": [1.0]})
    rows += report.record(operation("backward"), {"custom": [3.0], "PyTorch": [9.0]})
    text = report.render_tables(rows)
    tables = text.strip().split("\n\n")
    assert len(tables) == 2
    first = tables[0].splitlines()
    assert first[0].startswith("| size") and "reference (PyTorch) us" in first[0] and first[0].rstrip().endswith("reference % |")
    assert len(first) == 4                                   # header, rule, forward, backward
    assert len({len(line) for line in first}) == 1           # every line padded to the same width
    assert "| 2.00 " in first[2] and "| 8.00 " in first[2] and "| 400.0 " in first[2]
    assert "reference (Other) us" in tables[1] and "| 50.0 " in tables[1]


def test_save_report_writes_three_files(tmp_path):
    rows = report.record(operation(notes={"flops": 1.0}), {"custom": [2.0], "PyTorch": [8.0]})
    samples = [dict(size="B=1,T=512", dtype="bf16", operation="forward", samples_us={"custom": [2.0], "PyTorch": [8.0]})]
    text = report.save_report(tmp_path / "runtime", "mla", rows, samples, {"gpu": "test", "torch": "x"})
    assert (tmp_path / "runtime" / "mla.md").read_text() == text
    with open(tmp_path / "runtime" / "mla.csv", newline="") as handle:
        parsed = list(csv.DictReader(handle))
    assert parsed[0]["custom_us"] == "2.0" and parsed[0]["reference"] == "PyTorch"
    stored = json.loads((tmp_path / "runtime" / "mla_samples.json").read_text())
    assert stored["gpu"] == "test" and stored["samples"] == samples and "HIP graph replay" in stored["timing"]
    with pytest.raises(ValueError):
        report.save_report(tmp_path, "empty", [], [], {})


def harness(*arguments):
    return subprocess.run([sys.executable, "-m", "dscuda_amd.harness.run", *arguments], capture_output=True, text=True,
                          cwd=ROOT, timeout=300)


def test_entry_point_rejects_unknown_families_and_suites():
    assert harness("matmul").returncode == 2
    assert harness("mla", "--suite", "h100").returncode == 2


def test_entry_point_needs_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    result = harness("mla")
    assert result.returncode != 0 and "needs a GPU" in result.stderr


# ---- the PyTorch expressions run.py times and checks against, pinned on the CPU against the oracle ----------

def test_harness_reference_matches_the_oracle_for_causal_attention():
    import torch
    from dscuda_amd.harness import configs, run
    from oracle import attention_oracle as oracle
    q, k, v, scale = configs.mla_prefill_inputs(batch=2, seq=96, heads=3, seed=5)
    out, lse = run._sdpa(q, k, v, scale, causal=True)
    expected, expected_lse = oracle.causal_attention_forward(q, k, v, scale)
    assert out.shape == expected.shape and lse.shape == expected_lse.shape == (2, 3, 96)
    torch.testing.assert_close(out, expected.float(), atol=2e-5, rtol=1e-4)
    torch.testing.assert_close(lse, expected_lse, atol=2e-5, rtol=1e-5)


def test_harness_reference_broadcasts_shared_keys_and_masks_lengths():
    import torch
    from dscuda_amd.harness import configs, run
    from oracle import attention_oracle as oracle
    # grouped-query heads: 4 query heads on 2 key/value heads
    q, k, v, scale = configs.flash_forward_inputs(1, 64, 4, 2, 64, seed=3, factor=0.5)
    out, lse = run._sdpa(q, k, v, scale, causal=True)
    expected, expected_lse = oracle.causal_attention_forward(q, k.repeat_interleave(2, dim=2), v.repeat_interleave(2, dim=2), scale)
    torch.testing.assert_close(out, expected.float(), atol=2e-5, rtol=1e-4)
    torch.testing.assert_close(lse, expected_lse, atol=2e-5, rtol=1e-5)
    # decode: one query token per sequence against a shared 576-wide cache cut to per-sequence lengths
    q_lat, q_rope, latent, k_rope, scale = configs.mla_absorbed_inputs(3, 70, 5, query_tokens=1)
    lengths = torch.tensor([1, 37, 70], dtype=torch.int32)
    packed, cache = torch.cat((q_lat, q_rope), -1), torch.cat((latent, k_rope), -1)
    mask = (torch.arange(70)[None] < lengths[:, None])[:, None, None]
    out, lse = run._sdpa(packed, cache[:, :, None], cache[:, :, None, :512], scale, mask=mask)
    expected, expected_lse = oracle.mla_decode_unrounded(packed, cache, lengths, scale)
    torch.testing.assert_close(out, expected.float().reshape(out.shape), atol=2e-5, rtol=1e-4)
    torch.testing.assert_close(lse.reshape(-1), expected_lse.float().reshape(-1), atol=2e-5, rtol=1e-5)


def test_harness_check_uses_per_output_tolerances():
    import torch
    from dscuda_amd.harness import run
    expected = (torch.zeros(4), torch.zeros(4))
    run._close((torch.full((4,), 5e-3), torch.full((4,), 5e-5)), expected, (8e-3, 1e-4), (8e-3, 1e-4))
    with pytest.raises(AssertionError):
        run._close((torch.full((4,), 5e-3), torch.full((4,), 5e-3)), expected, (8e-3, 1e-4), (8e-3, 1e-4))
    with pytest.raises(AssertionError):
        run._close(torch.zeros(4), expected, 1e-2, 1e-2)      # one output where two are expected
