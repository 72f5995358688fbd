"""The reference harness's own acceptance bars at its own shapes, through the C-ABI.

The reference checks each operation with ``torch.testing.assert_close`` against the
bf16-rounded result of its PyTorch oracle (``benchmarks/common.py:58-65``):

* MLA forward and decode: O atol = rtol = 8e-3, LSE atol = rtol = 1e-4
  (``benchmarks/mla.py:103-105``);
* MLA backward: atol = rtol = 1e-2 against bf16-rounded autograd gradients
  (``benchmarks/mla.py:107-125``);
* flash forward: O atol = rtol = 1e-2, LSE atol 1e-4 / rtol 1e-5
  (``benchmarks/flash_attention.py:112-113``).

Inputs follow the reference's scaling (MLA 0.25 * N(0,1), dO 0.2 * N(0,1), flash
0.5 * N(0,1)); they come from a CPU generator instead of the reference's CUDA one."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce

pytestmark = pytest.mark.gpu


def _close(name, actual, expected, atol, rtol):
    torch.testing.assert_close(actual.cpu(), expected, atol=atol, rtol=rtol, msg=lambda m: f"{name}: {m}")


@pytest.mark.parametrize("batch,tokens,heads", configs.MLA_TEST_PREFILL + configs.MLA_FULL_PREFILL)
def test_mla_forward_and_backward_at_reference_bars(cuda, batch, tokens, heads):
    ql, qr, c, kr, scale = configs.mla_absorbed_inputs(batch, tokens, heads)
    mask = oracle.causal_mask(tokens)
    announce("reference bars: mla forward/backward", dict(B=batch, T=tokens, H=heads))
    out, lse = ops.mla_forward(ql.to(cuda), qr.to(cuda), c.to(cuda), kr.to(cuda), scale)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.mla_forward(ql, qr, c, kr, scale, mask)
    _close("O", out, expected, 8e-3, 8e-3)
    _close("LSE", lse, expected_lse, 1e-4, 1e-4)

    g = torch.Generator().manual_seed(2027)
    dout = (torch.randn(batch, tokens, heads, 512, generator=g) * 0.2).bfloat16()
    grads = ops.mla_backward(dout.to(cuda), expected.to(cuda), expected_lse.to(cuda), ql.to(cuda), qr.to(cuda),
                             c.to(cuda), kr.to(cuda), scale)
    torch.cuda.synchronize()
    # expected gradients the reference's way: autograd through the fp32 oracle, rounded to bf16
    leaves = [x.float().requires_grad_() for x in (ql, qr, c, kr)]
    unrounded, _ = oracle.mla_forward_unrounded(*leaves, scale, mask)
    reference = torch.autograd.grad(unrounded, leaves, dout.float())
    for name, actual, ref in zip(("dq_latent", "dq_rope", "dlatent", "dk_rope"), grads, reference):
        _close(name, actual, ref.bfloat16(), 1e-2, 1e-2)


@pytest.mark.parametrize("batch,tokens,heads", configs.MLA_TEST_DECODE + configs.MLA_FULL_DECODE)
def test_mla_decode_at_reference_bars(cuda, batch, tokens, heads):
    test_mode = (batch, tokens, heads) in configs.MLA_TEST_DECODE
    lengths = torch.tensor(configs.harness_decode_lengths(batch, tokens, test=test_mode), dtype=torch.int32)
    g = torch.Generator().manual_seed(2028)
    query = (torch.randn(batch, 1, heads, 576, generator=g) * 0.25).bfloat16()
    cache = (torch.randn(batch, tokens, 576, generator=g) * 0.25).bfloat16()
    scale = configs.c_float(576 ** -0.5)
    paged, table = configs.pack_cache(cache, 64)
    announce("reference bars: mla decode", dict(B=batch, KV=tokens, H=heads))
    out, lse = ops.mla_decode(query.to(cuda), paged.to(cuda), table.to(cuda), lengths.to(cuda), scale, splits=8)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.mla_decode_unrounded(query, cache, lengths, scale)
    _close("O", out, expected.bfloat16(), 8e-3, 8e-3)
    _close("LSE", lse, expected_lse, 1e-4, 1e-4)


@pytest.mark.parametrize("shape", configs.FLASH_TEST)
def test_flash_forward_at_reference_bars(cuda, shape):
    q, k, v, scale = configs.flash_forward_inputs(*shape, seed=2029, factor=0.5)
    announce("reference bars: flash forward", shape)
    out, lse = ops.flash_forward(q.to(cuda), k.to(cuda), v.to(cuda), scale)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.causal_attention_forward(q, k, v, scale)
    _close("O", out, expected.bfloat16(), 1e-2, 1e-2)
    _close("LSE", lse, expected_lse, 1e-4, 1e-5)
