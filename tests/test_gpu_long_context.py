"""GPU parity of the long-context workload (B=1, S=16384, H=128, 192/192/128, seed 4): forward and
recompute backward through the C-ABI at full size.  The fp32 oracle materialises one head's
16384 x 16384 score matrix at a time, so it is run on one sampled head; every head is covered by
size-independent properties (finite results, row 0 of O equals row 0 of V, the last key's dK/dV
rows depend on the last query alone)."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16, assert_close_lse

pytestmark = pytest.mark.gpu


def test_long_context_forward_and_backward_workload_5(cuda):
    q, k, v, dout, scale = configs.mla_long_context_inputs()
    batch, seq, heads, _ = q.shape
    checked = [77]
    sub = lambda t: t[:, :, checked]
    announce("mla_prefill_forward workload 5", tuple(q.shape))
    dq_, dk_, dv_, ddo = q.to(cuda), k.to(cuda), v.to(cuda), dout.to(cuda)
    out, lse = ops.mla_prefill_forward(dq_, dk_, dv_, scale)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.causal_attention_forward(sub(q), sub(k), sub(v), scale)
    assert_close_bf16("O", out[:, :, checked].cpu(), expected)
    assert_close_lse("LSE", lse[:, checked].cpu(), expected_lse)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    assert torch.equal(out[0, 0].cpu(), v[0, 0])   # a query that sees one key returns its value

    # backward from the oracle's saved tensors on the checked head, the kernel's own elsewhere
    saved_out = out.clone()
    saved_lse = lse.clone()
    saved_out[:, :, checked] = expected.bfloat16().to(cuda)
    saved_lse[:, checked] = expected_lse.to(cuda)
    announce("mla_prefill_backward workload 5")
    grads = ops.mla_prefill_backward(ddo, saved_out, saved_lse, dq_, dk_, dv_, scale)
    torch.cuda.synchronize()
    reference = oracle.attention_backward(sub(dout), expected.bfloat16(), expected_lse, sub(q), sub(k), sub(v), scale)
    for name, actual, wanted in zip(("dQ", "dK", "dV"), grads, reference):
        assert torch.isfinite(actual.float()).all(), name
        assert_close_bf16(name, actual[:, :, checked].cpu(), wanted)
    # the last key is seen by the last query only, with probability exp(s - lse): closed forms for every head
    last = seq - 1
    s_last = (q[0, last].float() * k[0, last].float()).sum(-1) * scale
    p_last = torch.exp(s_last - saved_lse[0, :, last].cpu())
    assert_close_bf16("dV last row", grads[2][0, last].cpu(), p_last[:, None] * dout[0, last].float())
