"""Seeded synthetic inputs of the five headline workloads and of the
reference harness's own test shapes.

Everything is drawn from a CPU ``torch.Generator`` so that the GPU box and the
development container see identical values, then rounded to bf16; an fp32
checker sees exactly the bf16-rounded values, the rule of
``benchmarks/mla.py:54``.  Scales are passed on as C floats
(``benchmarks/mla.py:55``).
"""

from __future__ import annotations

import math

import torch

from .common import c_float

MLA_RANK, MLA_ROPE = 512, 64

# reference test / benchmark shapes (benchmarks/mla.py:34-45, benchmarks/flash_attention.py:41-56)
MLA_TEST_PREFILL = [(1, 1, 1), (2, 17, 3), (1, 65, 4)]
MLA_TEST_DECODE = [(2, 23, 3), (3, 64, 16), (2, 65, 64), (3, 129, 128)]
MLA_FULL_PREFILL = [(1, 128, 8), (2, 257, 4), (1, 512, 8)]
MLA_FULL_DECODE = [(2, 1024, 16), (1, 256, 16), (4, 4096, 32)]
FLASH_TEST = [(1, 64, 2, 2, 128), (2, 64, 4, 2, 128), (1, 128, 4, 1, 128), (1, 256, 8, 8, 128)]


def _randn(generator, shape, factor=1.0):
    return (torch.randn(shape, generator=generator, dtype=torch.float32) * factor)


def apply_rope(x, theta=10000.0):
    """Rotate the last dimension of x [B,S,H,R] at positions 0..S-1 with the
    interleaved-pair convention: pairs (x[2i], x[2i+1]), freq_i = theta**(-2i/R)."""
    _, seq, _, width = x.shape
    half = width // 2
    freqs = theta ** (-torch.arange(half, dtype=torch.float64) * 2.0 / width)
    angles = torch.arange(seq, dtype=torch.float64)[:, None] * freqs[None]
    cos = angles.cos().float()[None, :, None, :]
    sin = angles.sin().float()[None, :, None, :]
    even, odd = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = even * cos - odd * sin
    out[..., 1::2] = even * sin + odd * cos
    return out


def flash_forward_inputs(batch=1, seq=512, q_heads=8, kv_heads=8, dim=64, seed=0, factor=1.0):
    """Workload 1: Q,K,V ~ N(0,1) seed 0, [B,T,H,D] memory layout, scale 1/sqrt(D)."""
    g = torch.Generator().manual_seed(seed)
    q = _randn(g, (batch, seq, q_heads, dim), factor).bfloat16()
    k = _randn(g, (batch, seq, kv_heads, dim), factor).bfloat16()
    v = _randn(g, (batch, seq, kv_heads, dim), factor).bfloat16()
    return q, k, v, c_float(dim ** -0.5)


def mla_prefill_inputs(batch=1, seq=4096, heads=128, nope=128, rope=64, dv=128, seed=1, rotate=True):
    """Workloads 2 and 5 (5: seq=16384, seed=4, rotate=False): Q,K [B,S,H,nope+rope],
    V [B,S,H,dv] ~ 0.5*N(0,1); rope slice rotated before bf16 rounding; scale 1/sqrt(nope+rope)."""
    g = torch.Generator().manual_seed(seed)
    dqk = nope + rope
    q = _randn(g, (batch, seq, heads, dqk), 0.5)
    k = _randn(g, (batch, seq, heads, dqk), 0.5)
    v = _randn(g, (batch, seq, heads, dv), 0.5)
    if rotate:
        q[..., nope:] = apply_rope(q[..., nope:])
        k[..., nope:] = apply_rope(k[..., nope:])
    return q.bfloat16(), k.bfloat16(), v.bfloat16(), c_float(dqk ** -0.5)


def mla_prefill_dout(batch=1, seq=4096, heads=128, dv=128, seed=2, factor=1.0):
    """Workload 3: dO ~ N(0,1) from seed 2."""
    g = torch.Generator().manual_seed(seed)
    return _randn(g, (batch, seq, heads, dv), factor).bfloat16()


def mla_long_context_inputs(batch=1, seq=16384, heads=128, nope=128, rope=64, dv=128, seed=4):
    """Workload 5: Q, K [B,S,H,192], V [B,S,H,128] ~ 0.5*N(0,1) and dO [B,S,H,128] ~ N(0,1), all from
    one generator seeded with 4, no rotation; scale 1/sqrt(192)."""
    g = torch.Generator().manual_seed(seed)
    dqk = nope + rope
    q = _randn(g, (batch, seq, heads, dqk), 0.5).bfloat16()
    k = _randn(g, (batch, seq, heads, dqk), 0.5).bfloat16()
    v = _randn(g, (batch, seq, heads, dv), 0.5).bfloat16()
    dout = _randn(g, (batch, seq, heads, dv), 1.0).bfloat16()
    return q, k, v, dout, c_float(dqk ** -0.5)


def decode_lengths(batch=64, low=1024, high=8192, seed=3):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(low, high + 1, (batch,), generator=g, dtype=torch.int64).to(torch.int32), g


def pack_cache(kv, page_size=64):
    """[B,N,W] -> ([B*pages,page,1,W] zero padded, identity int32 table); the
    packing of reference/python/mla.py:11-23."""
    batch, tokens, width = kv.shape
    pages = (tokens + page_size - 1) // page_size
    padded = torch.nn.functional.pad(kv, (0, 0, 0, pages * page_size - tokens))
    table = torch.arange(batch * pages, device=kv.device, dtype=torch.int32).reshape(batch, pages)
    return padded.reshape(batch * pages, page_size, 1, width).contiguous(), table


def mla_decode_inputs(batch=64, heads=128, low=1024, high=8192, seed=3, page_size=64):
    """Workload 4: lengths ~ U[low,high] from seed 3, query [B,1,H,576] and cache
    [B,max_len,576] ~ 0.5*N(0,1) from the same generator, packed to pages with an
    identity table, scale 1/sqrt(192).  Returns a dict; 'cache' is the contiguous
    form the checker consumes."""
    lengths, g = decode_lengths(batch, low, high, seed)
    width = MLA_RANK + MLA_ROPE
    max_len = int(lengths.max())
    query = _randn(g, (batch, 1, heads, width), 0.5).bfloat16()
    cache = _randn(g, (batch, max_len, width), 0.5).bfloat16()
    paged, table = pack_cache(cache, page_size)
    return dict(query=query, cache=cache, paged=paged, table=table, lengths=lengths,
                scale=c_float(192 ** -0.5), page_size=page_size)


def mla_absorbed_inputs(batch, tokens, heads, seed=2026, query_tokens=None, factor=0.25):
    """Inputs shaped like the reference harness's (benchmarks/mla.py:51-53):
    (q_lat [B,Q,H,512], q_rope [B,Q,H,64], latent [B,T,512], k_rope [B,T,64]) * 0.25."""
    g = torch.Generator().manual_seed(seed)
    q = tokens if query_tokens is None else query_tokens
    shapes = ((batch, q, heads, MLA_RANK), (batch, q, heads, MLA_ROPE), (batch, tokens, MLA_RANK),
              (batch, tokens, MLA_ROPE))
    tensors = tuple(_randn(g, shape, factor).bfloat16() for shape in shapes)
    return (*tensors, c_float((MLA_RANK + MLA_ROPE) ** -0.5))


def harness_decode_lengths(batch, tokens, test=True):
    """benchmarks/mla.py:58-61."""
    lengths = [max(1, tokens - i * tokens // (2 * batch)) for i in range(batch)]
    if test:
        lengths = [1] + lengths[1:-1] + [tokens]
    return lengths


# ---- algorithmic work (numerators of the roofline fractions) -----------------

def forward_flops(batch, heads, seq, dqk, dv):
    """Causal pair count S^2/2, two GEMMs."""
    return batch * heads * (seq * seq / 2) * 2 * (dqk + dv)


def backward_flops(batch, heads, seq, dqk, dv):
    """Five GEMMs (S, dP, dV, dQ, dK); recompute in the dQ pass is not counted."""
    return batch * heads * (seq * seq / 2) * 2 * (3 * dqk + 2 * dv)


def decode_bytes(total_tokens, batch, heads, rank=512, rope=64):
    width = rank + rope
    return total_tokens * width * 2 + batch * heads * (width * 2 + rank * 2 + 4)


def decode_flops(total_tokens, heads, rank=512, rope=64):
    return total_tokens * heads * 2 * (2 * rank + rope)
