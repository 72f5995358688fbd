"""Seeded random shapes through every entry point against the fp32 oracle: lengths around the tile sizes (32, 64,
128, 256), odd head counts, grouped heads, permuted pages of several sizes, split counts from 1 to 16."""

import random

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16, assert_close_lse

pytestmark = pytest.mark.gpu

SEQUENCES = [1, 2, 31, 63, 64, 65, 127, 129, 191, 200, 255, 257, 300, 449, 513]
TOKENS = [1, 2, 17, 31, 32, 33, 64, 65, 97, 129, 200, 257, 300]
ABSORBED_HEADS = [1, 2, 3, 5, 7, 8, 16, 20, 33, 48, 64, 100, 128]


def _randn(generator, shape, factor):
    return (torch.randn(shape, generator=generator) * factor).bfloat16()


@pytest.mark.parametrize("case", range(8))
def test_random_prefill(cuda, case):
    rnd = random.Random(100 + case)
    g = torch.Generator().manual_seed(100 + case)
    b, s, h = rnd.randint(1, 3), rnd.choice(SEQUENCES), rnd.randint(1, 9)
    announce("random prefill", dict(B=b, S=s, H=h))
    q, k, v = _randn(g, (b, s, h, 192), 0.5), _randn(g, (b, s, h, 192), 0.5), _randn(g, (b, s, h, 128), 0.5)
    dout = _randn(g, (b, s, h, 128), 1.0)
    scale = configs.c_float(192 ** -0.5)
    out, lse = ops.mla_prefill_forward(q.to(cuda), k.to(cuda), v.to(cuda), scale)
    expected, expected_lse = oracle.causal_attention_forward(q, k, v, scale)
    assert_close_bf16("O", out, expected)
    assert_close_lse("LSE", lse, expected_lse)
    saved = expected.bfloat16()
    grads = ops.mla_prefill_backward(dout.to(cuda), saved.to(cuda), expected_lse.to(cuda), q.to(cuda), k.to(cuda),
                                     v.to(cuda), scale)
    for name, actual, reference in zip(("dQ", "dK", "dV"), grads,
                                       oracle.attention_backward(dout, saved, expected_lse, q, k, v, scale)):
        assert_close_bf16(name, actual, reference)


@pytest.mark.parametrize("case", range(8))
def test_random_flash(cuda, case):
    rnd = random.Random(200 + case)
    g = torch.Generator().manual_seed(200 + case)
    d = rnd.choice([64, 128])
    kv_heads, group = rnd.randint(1, 4), rnd.choice([1, 2, 3, 4])
    b, t = rnd.randint(1, 3), 64 * rnd.randint(1, 9)   # the flash entry points take multiples of 64
    announce("random flash", dict(B=b, T=t, Hq=kv_heads * group, Hkv=kv_heads, D=d))
    q = _randn(g, (b, t, kv_heads * group, d), 0.5)
    k, v = _randn(g, (b, t, kv_heads, d), 0.5), _randn(g, (b, t, kv_heads, d), 0.5)
    dout = _randn(g, (b, t, kv_heads * group, d), 0.5)
    scale = configs.c_float(d ** -0.5)
    out, lse = ops.flash_forward(q.to(cuda), k.to(cuda), v.to(cuda), scale)
    expected, expected_lse = oracle.causal_attention_forward(q, k, v, scale)
    assert_close_bf16("O", out, expected)
    assert_close_lse("LSE", lse, expected_lse)
    saved = expected.bfloat16()
    grads = ops.flash_backward(dout.to(cuda), saved.to(cuda), expected_lse.to(cuda), q.to(cuda), k.to(cuda), v.to(cuda),
                               scale)
    for name, actual, reference in zip(("dQ", "dK", "dV"), grads,
                                       oracle.attention_backward(dout, saved, expected_lse, q, k, v, scale)):
        assert_close_bf16(name, actual, reference)


@pytest.mark.parametrize("case", range(8))
def test_random_absorbed(cuda, case):
    rnd = random.Random(300 + case)
    g = torch.Generator().manual_seed(300 + case)
    b, t, h = rnd.randint(1, 3), rnd.choice(TOKENS), rnd.choice(ABSORBED_HEADS)
    if t * h > 20000:
        h = max(1, 20000 // t)
    announce("random absorbed", dict(B=b, T=t, H=h))
    ql, qr = _randn(g, (b, t, h, 512), 0.25), _randn(g, (b, t, h, 64), 0.25)
    latent, kr = _randn(g, (b, t, 512), 0.25), _randn(g, (b, t, 64), 0.25)
    dout = _randn(g, (b, t, h, 512), 0.2 if h <= 32 else 0.05)
    scale = configs.c_float(576 ** -0.5)
    mask = oracle.causal_mask(t)
    out, lse = ops.mla_forward(ql.to(cuda), qr.to(cuda), latent.to(cuda), kr.to(cuda), scale)
    expected, expected_lse = oracle.mla_forward_unrounded(ql, qr, latent, kr, scale, mask)
    assert_close_bf16("O", out, expected, max_abs=8e-3)     # the reference's own bars (benchmarks/mla.py)
    assert_close_lse("LSE", lse, expected_lse, tol=1e-4)
    saved = expected.bfloat16()
    grads = ops.mla_backward(dout.to(cuda), saved.to(cuda), expected_lse.to(cuda), ql.to(cuda), qr.to(cuda),
                             latent.to(cuda), kr.to(cuda), scale)
    references = oracle.mla_backward_unrounded(dout, saved, expected_lse, ql, qr, latent, kr, scale, mask)
    for name, actual, reference in zip(("dq_latent", "dq_rope", "dlatent", "dk_rope"), grads, references):
        assert_close_bf16(name, actual, reference)


@pytest.mark.parametrize("case", range(10))
def test_random_decode(cuda, case):
    rnd = random.Random(400 + case)
    g = torch.Generator().manual_seed(400 + case)
    b, h = rnd.randint(1, 9), rnd.choice([1, 3, 16, 40, 64, 100, 128, 160])
    page = rnd.choice([16, 32, 64, 128])
    tokens = rnd.choice([1, 5, 63, 64, 65, 129, 300, 700, 1500])
    lengths = [rnd.randint(1, tokens) for _ in range(b)]
    splits = rnd.choice([1, 2, 3, 4, 8, 16])
    announce("random decode", dict(B=b, KV=tokens, H=h, page=page, lengths=lengths, splits=splits))
    query, cache = _randn(g, (b, 1, h, 576), 0.25), _randn(g, (b, tokens, 576), 0.25)
    scale = configs.c_float(576 ** -0.5)
    paged, table = configs.pack_cache(cache, page)
    order = torch.randperm(paged.shape[0], generator=g)
    inverse = torch.empty_like(order)
    inverse[order] = torch.arange(order.numel())
    paged, table = paged[order].contiguous(), inverse[table.long()].to(torch.int32)
    lengths_t = torch.tensor(lengths, dtype=torch.int32)
    out, lse = ops.mla_decode(query.to(cuda), paged.to(cuda), table.to(cuda), lengths_t.to(cuda), scale, splits=splits)
    expected, expected_lse = oracle.mla_decode_unrounded(query, cache, lengths_t, scale)
    assert_close_bf16("O", out, expected)
    assert_close_lse("LSE", lse, expected_lse)
