"""GPU parity of the causal flash-attention backward with grouped-query heads (dscuda_flash_backward) against the
fp32 oracle, whose grouped form is pinned to autograd in tests/test_oracle_pins.py.  The backward is fed the oracle's
bf16-rounded O and fp32 LSE, as the reference's harness does for its MLA backward (benchmarks/mla.py:68,113-117)."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16

pytestmark = pytest.mark.gpu


def _case(cuda, batch, seq, q_heads, kv_heads, dim, seed):
    q, k, v, scale = configs.flash_forward_inputs(batch, seq, q_heads, kv_heads, dim, seed=seed, factor=0.5)
    g = torch.Generator().manual_seed(seed + 500)
    dout = (torch.randn(batch, seq, q_heads, dim, generator=g) * 0.5).bfloat16()
    out_f, lse = oracle.causal_attention_forward(q, k, v, scale)
    out = out_f.bfloat16()
    announce("flash_backward", dict(B=batch, T=seq, Hq=q_heads, Hkv=kv_heads, D=dim))
    dq, dk, dv = ops.flash_backward(dout.to(cuda), out.to(cuda), lse.to(cuda), q.to(cuda), k.to(cuda), v.to(cuda), scale)
    torch.cuda.synchronize()
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    eq, ek, ev = oracle.attention_backward(dout, out, lse, q, k, v, scale)
    assert_close_bf16("dQ", dq.cpu(), eq)
    assert_close_bf16("dK", dk.cpu(), ek)
    assert_close_bf16("dV", dv.cpu(), ev)
    return dq, dk, dv


@pytest.mark.parametrize("batch,seq,q_heads,kv_heads,dim", [
    (1, 128, 4, 4, 128),      # MHA through the flash entry point
    (2, 192, 4, 2, 128),      # two query heads per key/value head
    (1, 257, 8, 1, 128),      # one shared key/value head, ragged length
    (1, 320, 6, 3, 64),       # D = 64
    (1, 64, 8, 2, 128),       # a single query tile: every tile of the walk is a diagonal one
    (2, 1, 4, 2, 128),
    (1, 1024, 8, 2, 128),     # the reference's quick-suite head counts
    (3, 200, 16, 2, 128),     # 6 pairs: the plain workgroup order (pairs not a multiple of 8)
    (2, 384, 32, 4, 128),     # 8 pairs: one pair at a time per XCD
])
def test_grouped_query_backward(cuda, batch, seq, q_heads, kv_heads, dim):
    _case(cuda, batch, seq, q_heads, kv_heads, dim, seed=61)


def test_grouped_query_backward_is_reproducible(cuda):
    """The sum over the query heads of a group is taken in a fixed order by one workgroup: two runs agree bit for bit."""
    first = _case(cuda, 1, 512, 8, 2, 128, seed=62)
    second = _case(cuda, 1, 512, 8, 2, 128, seed=62)
    for a, b in zip(first, second):
        assert torch.equal(a, b)


def test_shared_heads_equal_repeated_heads(cuda):
    """Grouped-query gradients are those of the same problem with K and V repeated per query head, summed over each
    group afterwards -- computed by the same kernels through the MHA path."""
    batch, seq, q_heads, kv_heads, dim = 1, 256, 8, 2, 128
    q, k, v, scale = configs.flash_forward_inputs(batch, seq, q_heads, kv_heads, dim, seed=63, factor=0.5)
    g = torch.Generator().manual_seed(64)
    dout = (torch.randn(batch, seq, q_heads, dim, generator=g) * 0.5).bfloat16()
    out, lse = ops.flash_forward(q.to(cuda), k.to(cuda), v.to(cuda), scale)
    grouped = ops.flash_backward(dout.to(cuda), out, lse, q.to(cuda), k.to(cuda), v.to(cuda), scale)
    group = q_heads // kv_heads
    k_wide, v_wide = k.repeat_interleave(group, dim=2).to(cuda), v.repeat_interleave(group, dim=2).to(cuda)
    wide = ops.flash_backward(dout.to(cuda), out, lse, q.to(cuda), k_wide, v_wide, scale)
    torch.cuda.synchronize()
    assert torch.equal(grouped[0], wide[0])       # dQ: the same arithmetic either way
    for shared, repeated in zip(grouped[1:], wide[1:]):
        summed = repeated.float().reshape(batch, seq, kv_heads, group, dim).sum(3)
        torch.testing.assert_close(shared.float(), summed, atol=3e-2, rtol=2e-2)


def test_flash_backward_rejects_bad_shapes(cuda):
    x = torch.zeros(1, 64, 3, 128, device=cuda, dtype=torch.bfloat16)
    kv = torch.zeros(1, 64, 2, 128, device=cuda, dtype=torch.bfloat16)
    lse = torch.zeros(1, 3, 64, device=cuda)
    with pytest.raises(RuntimeError, match="divisible"):
        ops.flash_backward(x, x, lse, x, kv, kv, 0.1, workspace=torch.zeros(16, device=cuda))
