"""GPU parity of the two per-head projections either side of absorbed attention (dscuda_mla_absorb_query,
dscuda_mla_unabsorb_output) against the fp32 oracle, through the C ABI.  The reference leaves these steps to its
caller (reference/python/sources.json:2)."""

import pytest
import torch

from dscuda_amd.harness import ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16

pytestmark = pytest.mark.gpu


def _weights(heads, seed):
    g = torch.Generator().manual_seed(seed)
    # wkv_b viewed [H, 128 + 128, 512]: the first half absorbs the query, the second un-absorbs the output
    wkv_b = (torch.randn(heads, 256, 512, generator=g) * 0.06).bfloat16()
    return wkv_b, g


@pytest.mark.parametrize("batch,seq,heads", [(1, 1, 1), (1, 31, 3), (2, 33, 16), (1, 513, 8), (1, 1100, 4), (3, 70, 128)])
def test_absorb_query(cuda, batch, seq, heads):
    wkv_b, g = _weights(heads, 41)
    query = (torch.randn(batch, seq, heads, 192, generator=g) * 0.5).bfloat16()   # nope columns 0..127
    announce("mla_absorb_query", dict(B=batch, S=seq, H=heads))
    device_weights = wkv_b.to(cuda)
    device_query = query.to(cuda)
    packed = torch.full((batch, seq, heads, 576), 7.0, device=cuda, dtype=torch.bfloat16)
    ops.mla_absorb_query(device_query[..., :128], device_weights[:, :128], out=packed[..., :512])
    torch.cuda.synchronize()
    expected = oracle.absorb_query(query[..., :128], wkv_b[:, :128])
    assert_close_bf16("q_latent", packed[..., :512].cpu(), expected)
    assert (packed[..., 512:].float() == 7.0).all()          # the rope columns of the packed query are untouched
    dense = ops.mla_absorb_query(device_query[..., :128].contiguous(), device_weights[:, :128].contiguous())
    torch.cuda.synchronize()
    assert torch.equal(dense.cpu(), packed[..., :512].cpu())  # layout does not change the result


@pytest.mark.parametrize("batch,seq,heads", [(1, 1, 1), (1, 31, 3), (2, 33, 16), (1, 513, 8), (1, 1100, 4), (3, 70, 128)])
def test_unabsorb_output(cuda, batch, seq, heads):
    wkv_b, g = _weights(heads, 43)
    latent_output = (torch.randn(batch, seq, heads, 512, generator=g) * 0.5).bfloat16()
    announce("mla_unabsorb_output", dict(B=batch, S=seq, H=heads))
    device_weights = wkv_b.to(cuda)
    out = ops.mla_unabsorb_output(latent_output.to(cuda), device_weights[:, 128:])
    torch.cuda.synchronize()
    expected = oracle.unabsorb_output(latent_output, wkv_b[:, 128:])
    assert_close_bf16("output", out.cpu(), expected)


def test_projections_compose_with_decode(cuda):
    """An absorbed decode step between the two projections equals per-head attention over the expanded keys and
    values (the identity that makes absorption valid), within bf16 rounding of the intermediate tensors."""
    batch, heads, length = 2, 16, 200
    wkv_b, g = _weights(heads, 47)
    q_nope = (torch.randn(batch, 1, heads, 128, generator=g) * 0.5).bfloat16()
    q_rope = (torch.randn(batch, 1, heads, 64, generator=g) * 0.5).bfloat16()
    cache = (torch.randn(batch, length, 576, generator=g) * 0.5).bfloat16()
    lengths = torch.tensor([length, 150], dtype=torch.int32)
    scale = 192 ** -0.5
    device_weights = wkv_b.to(cuda)
    packed = torch.empty(batch, 1, heads, 576, device=cuda, dtype=torch.bfloat16)
    packed[..., 512:] = q_rope.to(cuda)
    ops.mla_absorb_query(q_nope.to(cuda), device_weights[:, :128], out=packed[..., :512])
    paged, table = oracle.pack_cache(cache, 64)
    out_latent, _ = ops.mla_decode(packed, paged.to(cuda), table.to(cuda), lengths.to(cuda), scale, splits=4)
    out = ops.mla_unabsorb_output(out_latent, device_weights[:, 128:])
    torch.cuda.synchronize()
    # per-head attention in fp32 over k = [latent W_UK^T | rope], v = latent W_UV^T
    latent, rope = cache[..., :512].float(), cache[..., 512:].float()
    k_nope = torch.einsum("bsc,hdc->bshd", latent, wkv_b[:, :128].float())
    value = torch.einsum("bsc,hdc->bshd", latent, wkv_b[:, 128:].float())
    scores = (torch.einsum("bhd,bshd->bhs", q_nope[:, 0].float(), k_nope) +
              torch.einsum("bhr,bsr->bhs", q_rope[:, 0].float(), rope)) * scale
    visible = torch.arange(length)[None, None, :] < lengths[:, None, None]
    p = torch.softmax(scores.masked_fill(~visible, float("-inf")), dim=-1)
    expected = torch.einsum("bhs,bshd->bhd", p, value)[:, None]
    assert_close_bf16("decode between the projections", out.cpu(), expected)
