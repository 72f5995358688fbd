"""The reference's own prefill API (dscuda_mla_forward / dscuda_mla_backward) at the size the benchmark quotes,
B=1, T=4096, H=128: the paths the library chooses by itself at that size (row blocks of the unit stream in the
forward; the interval cut of the key gradients in the backward, taken when the rows outgrow the caches) against
the fp32 oracle, which works through the heads in chunks and sums the shared key / latent gradients over them."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16, assert_close_lse

pytestmark = pytest.mark.gpu

TOKENS, HEADS, CHUNK = 4096, 128, 8


def test_absorbed_forward_and_backward_at_the_benched_size(cuda):
    ql, qr, c, kr, scale = configs.mla_absorbed_inputs(1, TOKENS, HEADS)
    g = torch.Generator().manual_seed(91)
    # the shared gradients sum over 128 heads: dO is scaled so that the sums stay where half a bf16 step is
    # below the tolerance
    dout = (torch.randn(1, TOKENS, HEADS, 512, generator=g) * 0.05).bfloat16()
    mask = oracle.causal_mask(TOKENS)

    expected_out = torch.empty(1, TOKENS, HEADS, 512)
    expected_lse = torch.empty(1, HEADS, TOKENS)
    expected_dq = torch.empty(1, TOKENS, HEADS, 512)
    expected_dq_rope = torch.empty(1, TOKENS, HEADS, 64)
    expected_dlatent = torch.zeros(1, TOKENS, 512, dtype=torch.float64)
    expected_dk_rope = torch.zeros(1, TOKENS, 64, dtype=torch.float64)
    saved_out = torch.empty(1, TOKENS, HEADS, 512, dtype=torch.bfloat16)
    for first in range(0, HEADS, CHUNK):
        heads = slice(first, first + CHUNK)
        out, lse = oracle.mla_forward_unrounded(ql[:, :, heads], qr[:, :, heads], c, kr, scale, mask)
        expected_out[:, :, heads], expected_lse[:, heads] = out, lse
        saved_out[:, :, heads] = out.bfloat16()
        dq, dq_rope, dlatent, dk_rope = oracle.mla_backward_unrounded(
            dout[:, :, heads], saved_out[:, :, heads], lse, ql[:, :, heads], qr[:, :, heads], c, kr, scale, mask)
        expected_dq[:, :, heads], expected_dq_rope[:, :, heads] = dq, dq_rope
        expected_dlatent += dlatent.double()
        expected_dk_rope += dk_rope.double()
        del out, lse, dq, dq_rope, dlatent, dk_rope

    announce("mla_forward at the benched size", dict(B=1, T=TOKENS, H=HEADS))
    on_gpu = [x.to(cuda) for x in (ql, qr, c, kr)]
    out, lse = ops.mla_forward(*on_gpu, scale)
    torch.cuda.synchronize()
    assert_close_bf16("O", out, expected_out)
    assert_close_lse("LSE", lse, expected_lse)
    del out, lse

    announce("mla_backward at the benched size", dict(B=1, T=TOKENS, H=HEADS))
    grads = ops.mla_backward(dout.to(cuda), saved_out.to(cuda), expected_lse.to(cuda), *on_gpu, scale)
    torch.cuda.synchronize()
    expected = (expected_dq, expected_dq_rope, expected_dlatent.float(), expected_dk_rope.float())
    for name, actual, reference in zip(("dq_latent", "dq_rope", "dlatent", "dk_rope"), grads, expected):
        assert_close_bf16(name, actual.cpu(), reference)
