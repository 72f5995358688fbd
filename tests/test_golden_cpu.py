"""The CPU oracle reproduces the committed golden fixtures exactly (same
library, same thread-independent per-head loops), so a change to the oracle or
the fixtures shows up here before any GPU is involved."""

import torch

from oracle import attention_oracle as oracle
from tests.golden_data import load

TOL = 2e-6   # fp32 matmul summation order may differ with the host's thread count


def _close(a, b):
    return (a - b).abs().max().item() <= TOL


def test_flash_forward_fixture():
    d = load("flash_forward")
    out, lse = oracle.causal_attention_forward(d["q"], d["k"], d["v"], d["scale"])
    assert _close(out, d["out"]) and _close(lse, d["lse"])


def test_mla_prefill_fixture():
    d = load("mla_prefill")
    out, lse = oracle.causal_attention_forward(d["q"], d["k"], d["v"], d["scale"])
    assert _close(out, d["out"]) and _close(lse, d["lse"])
    assert torch.equal(out.bfloat16(), d["saved_out"])
    dq, dk, dv = oracle.attention_backward(d["dout"], d["saved_out"], d["lse"], d["q"], d["k"], d["v"], d["scale"])
    assert _close(dq, d["dq"]) and _close(dk, d["dk"]) and _close(dv, d["dv"])


def test_mla_absorbed_fixture():
    d = load("mla_absorbed")
    mask = oracle.causal_mask(d["ql"].shape[1])
    out, lse = oracle.mla_forward_unrounded(d["ql"], d["qr"], d["c"], d["kr"], d["scale"], mask)
    assert _close(out, d["out"]) and _close(lse, d["lse"])
    grads = oracle.mla_backward_unrounded(d["dout"], d["saved_out"], d["lse"], d["ql"], d["qr"], d["c"], d["kr"],
                                          d["scale"], mask)
    for actual, key in zip(grads, ("dql", "dqr", "dc", "dkr")):
        assert _close(actual, d[key]), key


def test_mla_decode_fixture():
    d = load("mla_decode")
    out, lse = oracle.mla_decode_unrounded(d["query"], d["cache"], d["lengths"], d["scale"])
    assert _close(out, d["out"]) and _close(lse, d["lse"])
    # row 0 has a single cached token: O is that token's latent, LSE its score
    assert torch.allclose(out[0, 0], d["cache"][0, 0, :512].float().expand(4, 512), atol=1e-6)
