"""Host-only checks of the runtime harness: the catalogue of workloads (dscuda_amd/harness/catalogue.py), the
sample bookkeeping of the timing (replay.py), the tables and report files (tables.py) and the argument handling of the
entry point (run.py) -- on numbers whose answers can be read off, without a GPU."""

import csv
import json
import subprocess
import sys
from pathlib import Path

import pytest

from dscuda_amd.harness import catalogue, configs, replay, tables

ROOT = Path(__file__).resolve().parents[1]


# ---- catalogue ------------------------------------------------------------------------------------------------

def test_test_mode_selects_the_reference_harness_shapes():
    mla = catalogue.select("mla", test=True)
    assert [w.shape for w in mla if w.operation == "forward"] == configs.MLA_TEST_PREFILL    # benchmarks/mla.py:36-37
    assert [w.shape for w in mla if w.operation == "backward"] == configs.MLA_TEST_PREFILL
    assert [w.shape for w in mla if w.operation == "decode"] == configs.MLA_TEST_DECODE      # benchmarks/mla.py:37-39
    assert [w.shape for w in catalogue.select("flash_attention", test=True)] == configs.FLASH_TEST


def test_suites_select_the_reference_harness_shapes():
    quick = catalogue.select("mla", "quick")
    assert {(w.operation, w.shape) for w in quick} == {("forward", (1, 128, 8)), ("backward", (1, 128, 8)),
                                                       ("decode", (2, 1024, 16))}           # benchmarks/mla.py:34
    full = catalogue.select("mla", "full")
    assert {w.shape for w in full if w.operation == "decode"} == {(2, 1024, 16), (1, 256, 16), (4, 4096, 32)}
    h100 = catalogue.select("mla", "h100")                                                   # benchmarks/mla.py:40-42
    assert [w.shape for w in h100] == [(1, 1024, 64), (4, 4096, 64), (4, 4096, 128), (8, 8192, 128)]
    assert all(w.operation == "decode" for w in h100)
    assert len(catalogue.select("flash_attention", "full")) == 2 * 5 * 3                    # flash_attention.py:50-56
    assert [w.shape for w in catalogue.select("flash_attention", "quick")] == [(1, 512, 8, kv, 128) for kv in (8, 2, 1)]
    assert catalogue.select("mla", "full", operation="decode") == [w for w in full if w.operation == "decode"]
    assert catalogue.select("mla", "h100", operation="backward") == []
    with pytest.raises(ValueError):
        catalogue.select("matmul")
    with pytest.raises(ValueError):
        catalogue.select("mla", "everything")


def test_labels_follow_the_reference_tables():
    assert catalogue.Workload("flash_attention", "forward", (1, 512, 8, 2, 128)).label == "B=1,T=512,Hq=8,Hkv=2,D=128"
    assert catalogue.Workload("mla", "forward", (2, 257, 4)).label == "B=2,Q=257,KV=257,H=4,C=512,RoPE=64"
    decode = catalogue.Workload("mla", "decode", (2, 1024, 16)).label                        # benchmarks/mla.py:100-102
    assert decode == "B=2,Q=1,KV=1024,H=16,C=512,RoPE=64,lengths=(1024, 768),page=64,custom_splits=8"
    tested = catalogue.Workload("mla", "decode", (3, 64, 16), test=True).label               # benchmarks/mla.py:59-60
    assert "lengths=(1, 54, 64)" in tested


# ---- replay bookkeeping ----------------------------------------------------------------------------------------

def test_replays_fill_the_sample_window():
    assert replay.replays_per_sample(20, 0.5) == 40
    assert replay.replays_per_sample(20, 0.3) == 67             # rounded up
    assert replay.replays_per_sample(20, 100.0) == 1            # never zero
    assert replay.replays_per_sample(20, 0.0) == replay.MOST_REPLAYS   # a zero measurement neither divides by zero nor runs forever


def test_every_backend_starts_a_trial_in_turn():
    orders = replay.starting_orders(["custom", "PyTorch"], 4)
    assert orders == [["custom", "PyTorch"], ["PyTorch", "custom"], ["custom", "PyTorch"], ["PyTorch", "custom"]]
    three = replay.starting_orders(["a", "b", "c"], 3)
    assert [order[0] for order in three] == ["a", "b", "c"] and all(sorted(order) == ["a", "b", "c"] for order in three)


def test_settings_reject_nonsense():
    replay.Settings(10, 0, 5, 1)
    for bad in ((0, 1000, 20, 9), (10, 1000, 0, 9), (10, 1000, 20, 0), (10, -1, 20, 9)):
        with pytest.raises(ValueError):
            replay.Settings(*bad)


# ---- tables -----------------------------------------------------------------------------------------------------

def test_rows_carry_medians_and_the_reference_percent():
    rows = tables.summarise("B=1,T=512", "bf16", "forward", {"custom": [10.0, 30.0, 20.0], "PyTorch": [100.0, 50.0, 60.0]})
    assert rows == [tables.Row("B=1,T=512", "bf16", "forward", 20.0, "PyTorch", 60.0, pytest.approx(300.0))]


def test_a_custom_only_operation_keeps_its_time():
    rows = tables.summarise("B=1,T=512", "bf16", "forward", {"custom": [4.0, 6.0]})
    assert rows == [tables.Row("B=1,T=512", "bf16", "forward", 5.0, "none", None, None)]


def test_two_references_give_two_rows_and_two_tables():
    rows = tables.summarise("s", "bf16", "forward", {"custom": [2.0], "PyTorch": [8.0], "Other": [1.0]})
    assert [(row.reference, row.reference_pct) for row in rows] == [("PyTorch", 400.0), ("Other", 50.0)]
    rows += tables.summarise("s", "bf16", "backward", {"custom": [3.0], "PyTorch": [9.0]})
    parts = tables.markdown(rows).strip().split("\n\n")
    assert len(parts) == 2
    first = parts[0].splitlines()
    assert first[0].startswith("| size") and "reference (PyTorch) us" in first[0] and first[0].rstrip().endswith("reference % |")
    assert len(first) == 4                                   # header, rule, forward, backward
    assert len({len(line) for line in first}) == 1           # every line padded to the same width
    assert set(first[1]) <= set("|- ")
    assert "| 2.00 " in first[2] and "| 8.00 " in first[2] and "| 400.0 " in first[2]
    assert "reference (Other) us" in parts[1] and "| 50.0 " in parts[1]


def test_a_missing_reference_prints_dashes():
    text = tables.markdown(tables.summarise("s", "bf16", "decode", {"custom": [7.0]}))
    assert "reference (none) us" in text and text.count("—") == 2


def test_write_leaves_three_files(tmp_path):
    timings = {"custom": [2.0], "PyTorch": [8.0]}
    rows = tables.summarise("B=1,T=512", "bf16", "forward", timings)
    samples = [dict(size="B=1,T=512", dtype="bf16", operation="forward", samples_us=timings, flops=1.0)]
    text = tables.write(tmp_path / "runtime", "mla", rows, samples, {"gpu": "test", "torch": "x"})
    assert (tmp_path / "runtime" / "mla.md").read_text() == text
    with open(tmp_path / "runtime" / "mla.csv", newline="") as handle:
        parsed = list(csv.DictReader(handle))
    assert list(parsed[0]) == list(tables.CSV_FIELDS)        # the reference's column names (benchmarks/common.py:144-149)
    assert parsed[0]["custom_us"] == "2.0" and parsed[0]["reference"] == "PyTorch" and parsed[0]["reference_pct"] == "400.0"
    stored = json.loads((tmp_path / "runtime" / "mla_samples.json").read_text())
    assert stored["gpu"] == "test" and stored["samples"] == samples and "HIP graph replay" in stored["timing"]
    with pytest.raises(ValueError):
        tables.write(tmp_path, "empty", [], [], {})


# ---- entry point --------------------------------------------------------------------------------------------------

def harness(*arguments):
    return subprocess.run([sys.executable, "-m", "dscuda_amd.harness.run", *arguments], capture_output=True, text=True,
                          cwd=ROOT, timeout=300)


def test_entry_point_rejects_what_it_cannot_run():
    assert harness("matmul").returncode == 2
    assert harness("mla", "--suite", "everything").returncode == 2
    missing = harness("mla", "--reference", "flashmla")
    assert missing.returncode == 2 and "does not exist on this platform" in missing.stderr
    assert harness("mla", "--test", "--reference", "none").returncode == 2
    assert harness("mla", "--trials", "0").returncode == 2


def test_entry_point_needs_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    result = harness("mla", "--suite", "h100")
    assert result.returncode != 0 and "needs a GPU" in result.stderr


def test_the_benchmark_measures_one_gpu_only():
    result = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                            cwd=ROOT, timeout=120)
    assert result.returncode != 0
    assert "one GPU" in result.stdout + result.stderr and result.stdout.count("{") == 0


# ---- the PyTorch expressions the harness times and checks against, pinned on the CPU against the oracle -----------

def test_harness_reference_matches_the_oracle_for_causal_attention():
    import torch
    from oracle import attention_oracle as oracle
    q, k, v, scale = configs.mla_prefill_inputs(batch=2, seq=96, heads=3, seed=5)
    out, lse = catalogue._attention(q, k, v, scale, causal=True)
    expected, expected_lse = oracle.causal_attention_forward(q, k, v, scale)
    assert out.shape == expected.shape and lse.shape == expected_lse.shape == (2, 3, 96)
    torch.testing.assert_close(out, expected.float(), atol=2e-5, rtol=1e-4)
    torch.testing.assert_close(lse, expected_lse, atol=2e-5, rtol=1e-5)


def test_harness_reference_broadcasts_shared_keys_and_masks_lengths():
    import torch
    from oracle import attention_oracle as oracle
    # grouped-query heads: 4 query heads on 2 key/value heads
    q, k, v, scale = configs.flash_forward_inputs(1, 64, 4, 2, 64, seed=3, factor=0.5)
    out, lse = catalogue._attention(q, k, v, scale, causal=True)
    expected, expected_lse = oracle.causal_attention_forward(q, k.repeat_interleave(2, dim=2), v.repeat_interleave(2, dim=2), scale)
    torch.testing.assert_close(out, expected.float(), atol=2e-5, rtol=1e-4)
    torch.testing.assert_close(lse, expected_lse, atol=2e-5, rtol=1e-5)
    # decode: one query token per sequence against a shared 576-wide cache cut to per-sequence lengths
    q_lat, q_rope, latent, k_rope, scale = configs.mla_absorbed_inputs(3, 70, 5, query_tokens=1)
    lengths = torch.tensor([1, 37, 70], dtype=torch.int32)
    packed, cache = torch.cat((q_lat, q_rope), -1), torch.cat((latent, k_rope), -1)
    mask = (torch.arange(70)[None] < lengths[:, None])[:, None, None]
    out, lse = catalogue._attention(packed, cache[:, :, None], cache[:, :, None, :512], scale, mask=mask)
    expected, expected_lse = oracle.mla_decode_unrounded(packed, cache, lengths, scale)
    torch.testing.assert_close(out, expected.float().reshape(out.shape), atol=2e-5, rtol=1e-4)
    torch.testing.assert_close(lse.reshape(-1), expected_lse.float().reshape(-1), atol=2e-5, rtol=1e-5)


def test_harness_gradients_match_the_oracle():
    import torch
    from oracle import attention_oracle as oracle
    q, k, v, scale = configs.mla_prefill_inputs(batch=1, seq=80, heads=2, seed=6)
    dout = configs.mla_prefill_dout(1, 80, 2, 128, seed=7)
    got = catalogue._gradients(lambda a, b, c: catalogue._attention(a, b, c, scale, causal=True), (q, k, v), dout)
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    expected = oracle.attention_backward(dout, out, lse, q, k, v, scale)
    for a, b in zip(got, expected):
        torch.testing.assert_close(a, b.float(), atol=2e-4, rtol=1e-3)


def test_bound_workloads_compare_with_per_output_tolerances():
    import torch
    workload = catalogue.Workload("mla", "forward", (1, 1, 1))
    bound = catalogue.Bound(workload, {}, expected=(torch.zeros(4), torch.zeros(4)), tolerance=((8e-3, 8e-3), (1e-4, 1e-4)))
    bound.verify("custom", (torch.full((4,), 5e-3), torch.full((4,), 5e-5)))
    with pytest.raises(AssertionError):
        bound.verify("custom", (torch.full((4,), 5e-3), torch.full((4,), 5e-3)))
    with pytest.raises(AssertionError):
        bound.verify("custom", (torch.zeros(4),))
    catalogue.Bound(workload, {}).verify("custom", (torch.ones(1),))   # nothing to compare with: nothing to fail
