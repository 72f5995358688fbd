"""Every gradient and output row has one writer and every sum a fixed order (the reference's rule for its
kernels, kernels/attention/mla/sm89.cu:2): repeated calls on the same inputs agree bit for bit.  Sizes are chosen
so that the work is cut across many workgroups (ranges and intervals of the absorbed key gradients, split decode
walks, several key blocks per head) and the calls alternate with other work on the same buffers."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from tests.parity import announce

pytestmark = pytest.mark.gpu


def _randn(cuda, generator, shape, factor):
    return (torch.randn(shape, device=cuda, generator=generator) * factor).bfloat16()


@pytest.mark.parametrize("batch,tokens,heads", [(1, 2048, 32), (2, 700, 128), (1, 333, 5)])
def test_absorbed_prefill_is_reproducible(cuda, batch, tokens, heads):
    g = torch.Generator(device=cuda).manual_seed(5)
    ql, qr = _randn(cuda, g, (batch, tokens, heads, 512), 0.25), _randn(cuda, g, (batch, tokens, heads, 64), 0.25)
    latent, kr = _randn(cuda, g, (batch, tokens, 512), 0.25), _randn(cuda, g, (batch, tokens, 64), 0.25)
    dout = _randn(cuda, g, (batch, tokens, heads, 512), 0.1)
    scale = configs.c_float(576 ** -0.5)
    announce("mla_forward / mla_backward twice", dict(B=batch, T=tokens, H=heads))
    out, lse = ops.mla_forward(ql, qr, latent, kr, scale)
    first = [x.clone() for x in ops.mla_backward(dout, out, lse, ql, qr, latent, kr, scale)]
    out2, lse2 = ops.mla_forward(ql, qr, latent, kr, scale)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    grads = tuple(torch.full_like(x, 7.0) for x in first)   # the scratch use of the gradient buffers starts from other contents
    for _ in range(2):
        ops.mla_backward(dout, out, lse, ql, qr, latent, kr, scale, grads)
        torch.cuda.synchronize()
        for name, a, b in zip(("dq_latent", "dq_rope", "dlatent", "dk_rope"), first, grads):
            assert torch.equal(a, b), name


@pytest.mark.parametrize("batch,seq,heads", [(1, 1536, 16), (2, 449, 6)])
def test_prefill_is_reproducible(cuda, batch, seq, heads):
    g = torch.Generator(device=cuda).manual_seed(6)
    q, k = _randn(cuda, g, (batch, seq, heads, 192), 0.5), _randn(cuda, g, (batch, seq, heads, 192), 0.5)
    v, dout = _randn(cuda, g, (batch, seq, heads, 128), 0.5), _randn(cuda, g, (batch, seq, heads, 128), 1.0)
    scale = configs.c_float(192 ** -0.5)
    announce("mla_prefill_forward / _backward twice", dict(B=batch, S=seq, H=heads))
    out, lse = ops.mla_prefill_forward(q, k, v, scale)
    out2, lse2 = ops.mla_prefill_forward(q, k, v, scale)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    first = [x.clone() for x in ops.mla_prefill_backward(dout, out, lse, q, k, v, scale)]
    workspace = ops.mla_prefill_backward_workspace(batch, seq, heads, 192, 128, cuda)
    workspace.fill_(3.0)
    again = ops.mla_prefill_backward(dout, out, lse, q, k, v, scale, workspace)
    torch.cuda.synchronize()
    for name, a, b in zip(("dQ", "dK", "dV"), first, again):
        assert torch.equal(a, b), name
