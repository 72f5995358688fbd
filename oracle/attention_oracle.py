"""CPU oracle for the attention hot path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  Nothing in ``dscuda_amd`` imports it and the product path raises
when its HIP libraries are missing instead of falling back to this code.

It restates, in plain unfused fp32 PyTorch (fp64 when the caller passes
fp64 tensors), the mathematics the reference defines for this path:

* absorbed MLA forward / analytic backward / page packing follow
  ``reference/python/mla.py:11-57``;
* the precision rule (compute in fp32 unless the input already is wider)
  follows ``reference/python/attention.py:6-7`` and ``mla.py:6-8``;
* causal flash attention with GQA expansion and natural-log LSE follows
  ``benchmarks/flash_attention.py:70-77``;
* the decode length mask follows ``benchmarks/mla.py:62-66``;
* the decode workspace size follows ``kernels/attention/mla/sm89.cu:539-541``.

The per-head (128 nope + 64 rope | 128 v) prefill forward/backward named by
the headline configurations has no counterpart in the reference; its oracle
is textbook causal attention with ``d_v != d_qk`` in the same style.  The
two per-head projections either side of absorbed attention are likewise
outside the reference (``reference/python/sources.json:2``); their oracle is
one einsum each.  Rotary embedding is left to the caller by the reference as
well (same line); ``apply_rope`` states DeepSeek-V3's convention as a complex
multiplication.

How each function is pinned (see ``tests/test_oracle_pins.py``):

=====================  =====================================================
function               pins
=====================  =====================================================
causal_attention_*     ``torch.nn.functional.scaled_dot_product_attention``
                       (library routine), fp64 triple-loop brute force,
                       row-0 / shift-invariance / sum-to-one invariants,
                       GQA == repeat_interleave MHA
attention_backward     ``torch.autograd.grad`` through the forward (the
                       way the reference builds its expected gradients,
                       ``benchmarks/mla.py:108-110``), fp64 central finite
                       differences, ``sum_k dS = 0``
mla_forward            equals MQA attention on concatenated [latent|rope]
                       via SDPA; closed form of the constant fill in
                       ``benchmarks/attention/benchmark_mla.cu:38-47``
mla_backward           autograd through mla_forward; closed form of the
                       same constant fill with dO = 2**-6
mla_decode             SDPA with a length mask; equals row T-1 of the
                       causal prefill when len == T; closed form of
                       ``benchmark_mla_decode.cu:42-48``
pack_cache             closed form (identity table, zero padding)
apply_rope             closed forms: the unit pair (1, 0) at position p becomes
                       (cos, sin) of p * theta^(-2i/R); position 0 is the
                       identity; R = 2 leaves the single angle p; rotations
                       compose (p then q == p + q); relative-position
                       property of the rotated dot product; a half-split
                       pairing, a reversed direction and a -i/R exponent
                       each fail those checks
absorb_query,          fp64 triple-loop brute force; the identity absorption
unabsorb_output        rests on: scores and outputs of per-head attention
                       over k_nope = latent W_UK^T, v = latent W_UV^T equal
                       those of absorbed attention between the two
                       projections (a transposed or swapped weight fails it)
=====================  =====================================================

No function here is "parity unpinned".  The reference holds no golden
vectors for this path (its tests draw inputs from the CUDA generator), so the
fixtures under ``tests/golden`` are produced by this module after the pins
above pass.
"""

from __future__ import annotations

import math

import torch


def _compute(tensor: torch.Tensor) -> torch.Tensor:
    """fp32 unless the tensor is already >= 4 bytes wide (reference/python/mla.py:6-8)."""
    return tensor if tensor.element_size() >= 4 else tensor.float()


# --------------------------------------------------------------------------
# causal attention, [B, S, H, D] layout  (benchmarks/flash_attention.py:70-77)
# --------------------------------------------------------------------------

def causal_attention_forward(query, key, value, scale, heads=None):
    """O = softmax_causal(Q K^T * scale) V and LSE = ln sum exp (natural log).

    query [B,S,Hq,Dqk]; key [B,S,Hkv,Dqk]; value [B,S,Hkv,Dv]; Hq % Hkv == 0,
    query head h reads kv head h // (Hq/Hkv) (``repeat_interleave`` in
    benchmarks/flash_attention.py:72-74).  Returns (O [B,S,len(heads),Dv]
    unrounded, LSE [B,len(heads),S]) in the compute dtype.  ``heads`` selects
    a subset of query heads so that large shapes can be spot-checked; the
    score matrix is only ever materialised for one head at a time.
    """
    query, key, value = map(_compute, (query, key, value))
    batch, seq, q_heads, _ = query.shape
    kv_heads = key.shape[2]
    group = q_heads // kv_heads
    heads = list(range(q_heads)) if heads is None else list(heads)
    mask = torch.ones(seq, seq, dtype=torch.bool).tril()
    out = torch.empty(batch, seq, len(heads), value.shape[-1], dtype=query.dtype)
    lse = torch.empty(batch, len(heads), seq, dtype=query.dtype)
    for b in range(batch):
        for i, h in enumerate(heads):
            q = query[b, :, h]
            k = key[b, :, h // group]
            v = value[b, :, h // group]
            scores = (q @ k.transpose(0, 1) * scale).masked_fill(~mask, -math.inf)
            row_lse = scores.logsumexp(-1)
            out[b, :, i] = (scores - row_lse[:, None]).exp() @ v
            lse[b, i] = row_lse
    return out, lse


def attention_backward(dout, out, lse, query, key, value, scale, heads=None):
    """Analytic gradients of causal attention from saved O and LSE.

    Same recompute structure as reference/python/mla.py:42-57 with per-head
    K/V:  P = exp(S - LSE);  dP = dO V^T;  delta = sum_c dO*O;
    dS = P (dP - delta) scale;  dQ = dS K;  dK = dS^T Q;  dV = P^T dO.
    Grouped-query heads (Hq a multiple of Hkv, query head h reads kv head
    h // (Hq/Hkv) as in the forward): dK and dV of a kv head are the sums over
    the query heads of its group; ``heads`` must then be None.  Returns
    unrounded (dQ [B,S,heads,Dqk], dK [B,S,Hkv or heads,Dqk], dV likewise).
    """
    dout, out, query, key, value = map(_compute, (dout, out, query, key, value))
    lse = _compute(lse)
    batch, seq, q_heads, _ = query.shape
    kv_heads = key.shape[2]
    assert q_heads % kv_heads == 0, "query heads must be a multiple of key/value heads"
    group = q_heads // kv_heads
    assert group == 1 or heads is None, "a head subset is only defined for the MHA form"
    heads = list(range(q_heads)) if heads is None else list(heads)
    mask = torch.ones(seq, seq, dtype=torch.bool).tril()
    dq = torch.empty(batch, seq, len(heads), query.shape[-1], dtype=query.dtype)
    kv_count = len(heads) if group == 1 else kv_heads
    dk = torch.zeros(batch, seq, kv_count, query.shape[-1], dtype=query.dtype)
    dv = torch.zeros(batch, seq, kv_count, value.shape[-1], dtype=query.dtype)
    for b in range(batch):
        for i, h in enumerate(heads):
            shared = h // group
            q, k, v = query[b, :, h], key[b, :, shared], value[b, :, shared]
            do, o = dout[b, :, h], out[b, :, h]
            scores = (q @ k.transpose(0, 1) * scale).masked_fill(~mask, -math.inf)
            prob = (scores - lse[b, h][:, None]).exp()
            dprob = do @ v.transpose(0, 1)
            delta = (do * o).sum(-1, keepdim=True)
            dscore = prob * (dprob - delta) * scale
            dq[b, :, i] = dscore @ k
            target = i if group == 1 else shared
            dk[b, :, target] += dscore.transpose(0, 1) @ q
            dv[b, :, target] += prob.transpose(0, 1) @ do
    return dq, dk, dv


# --------------------------------------------------------------------------
# absorbed MLA  (reference/python/mla.py)
# --------------------------------------------------------------------------

def pack_cache(kv, page_size=64):
    """[B,N,W] -> ([B*pages, page, 1, W] zero padded, identity table) (mla.py:11-23)."""
    batch, tokens, width = kv.shape
    pages = (tokens + page_size - 1) // page_size
    padded = torch.zeros(batch, pages * page_size, width, dtype=kv.dtype)
    padded[:, :tokens] = kv
    table = torch.arange(batch * pages, dtype=torch.int32).reshape(batch, pages)
    return padded.reshape(batch * pages, page_size, 1, width).contiguous(), table


def causal_mask(tokens):
    return torch.ones(tokens, tokens, dtype=torch.bool).tril()


def length_mask(lengths, tokens):
    """[B,1,1,T] mask, key t visible iff t < len[b] (benchmarks/mla.py:62-66)."""
    lengths = torch.as_tensor(lengths)
    return (torch.arange(tokens)[None] < lengths[:, None])[:, None, None]


def _scores(query, query_rope, latent, key_rope, scale, mask):
    # mla.py:26-29: latent and rope parts contract separately, one shared KV head.
    score = (torch.einsum("bqhc,bkc->bhqk", query, latent)
             + torch.einsum("bqhr,bkr->bhqk", query_rope, key_rope)) * scale
    return score.masked_fill(~mask, -math.inf)


def mla_forward_unrounded(query, query_rope, latent, key_rope, scale, mask):
    """mla.py:32-39 without the final bf16 rounding: (O fp32 [B,Q,H,C], LSE [B,H,Q])."""
    query, query_rope, latent, key_rope = map(_compute, (query, query_rope, latent, key_rope))
    score = _scores(query, query_rope, latent, key_rope, scale, mask)
    lse = score.logsumexp(dim=-1)
    prob = (score - lse.unsqueeze(-1)).exp()
    out = torch.einsum("bhqk,bkc->bqhc", prob, latent)
    return out.contiguous(), lse.contiguous()


def mla_forward(query, query_rope, latent, key_rope, scale, mask):
    """Same return convention as the reference: bf16 O, fp32 LSE (mla.py:39)."""
    out, lse = mla_forward_unrounded(query, query_rope, latent, key_rope, scale, mask)
    return out.bfloat16().contiguous(), lse


def mla_backward_unrounded(dout, output, lse, query, query_rope, latent, key_rope, scale, mask):
    """mla.py:42-57 without the final bf16 rounding."""
    dout, output, query, query_rope, latent, key_rope = map(
        _compute, (dout, output, query, query_rope, latent, key_rope))
    score = _scores(query, query_rope, latent, key_rope, scale, mask)
    prob = (score - lse.unsqueeze(-1)).exp()
    dprob = torch.einsum("bqhc,bkc->bhqk", dout, latent)
    delta = (dout * output).sum(dim=-1).transpose(1, 2).unsqueeze(-1)
    dscore = prob * (dprob - delta) * scale
    dquery = torch.einsum("bhqk,bkc->bqhc", dscore, latent)
    dquery_rope = torch.einsum("bhqk,bkr->bqhr", dscore, key_rope)
    # the shared latent receives the key-path and the value-path gradient (mla.py:52-54)
    dlatent = (torch.einsum("bhqk,bqhc->bkc", dscore, query)
               + torch.einsum("bhqk,bqhc->bkc", prob, dout))
    dkey_rope = torch.einsum("bhqk,bqhr->bkr", dscore, query_rope)
    return tuple(t.contiguous() for t in (dquery, dquery_rope, dlatent, dkey_rope))


def mla_backward(dout, output, lse, query, query_rope, latent, key_rope, scale, mask):
    return tuple(t.bfloat16().contiguous() for t in mla_backward_unrounded(
        dout, output, lse, query, query_rope, latent, key_rope, scale, mask))


def mla_decode_unrounded(packed_query, cache, lengths, scale, rank=512):
    """One query token per sequence over ``lengths[b]`` cached tokens.

    packed_query [B,1,H,rank+rope]; cache [B,N,rank+rope] (contiguous, before
    page packing); lengths [B] (>= 1).  The decode is the absorbed forward with
    a length mask instead of the causal one (benchmarks/mla.py:62-67).
    Returns (O fp32 [B,1,H,rank], LSE [B,H,1]).
    """
    tokens = cache.shape[1]
    mask = length_mask(lengths, tokens)
    return mla_forward_unrounded(
        packed_query[..., :rank], packed_query[..., rank:],
        cache[..., :rank], cache[..., rank:], scale, mask)


def decode_workspace_elements(batch, heads, splits, rank):
    """kernels/attention/mla/sm89.cu:539-541."""
    return batch * heads * splits * (rank + 2)


# --------------------------------------------------------------------------
# error metrics used by every parity test
# --------------------------------------------------------------------------

def error_stats(actual, expected):
    """(max-abs, mean-abs) of actual - expected, both taken in fp64."""
    diff = (actual.double() - expected.double()).abs()
    return diff.max().item(), diff.mean().item()


def absorb_query(query_nope, w_uk):
    """q_latent[..., h, c] = sum_d q_nope[..., h, d] * w_uk[h, d, c] in fp32: the step before absorbed attention that
    the reference leaves to its caller (reference/python/sources.json:2).  Operand order as in the absorbed path of
    DeepSeek-V3's inference/model.py (q_nope times the first 128 rows per head of wkv_b)."""
    return torch.einsum("...hd,hdc->...hc", _compute(query_nope), _compute(w_uk))


def unabsorb_output(output_latent, w_uv):
    """out[..., h, d] = sum_c output_latent[..., h, c] * w_uv[h, d, c] in fp32: the step after absorbed attention
    (the latent output times the last 128 rows per head of wkv_b, same source)."""
    return torch.einsum("...hc,hdc->...hd", _compute(output_latent), _compute(w_uv))


def apply_rope(x, theta=10000.0, start=0):
    """Rotary position embedding of the last dimension of x [B, S, H, R], positions start .. start + S - 1, in the
    convention of DeepSeek-V3's ``apply_rotary_emb``: consecutive columns (2i, 2i + 1) are the real and imaginary
    part of one complex number, multiplied by ``exp(1j * position * theta ** (-2i / R))``.  The reference leaves this
    step to its caller (reference/python/sources.json:2), so the convention is this build's choice; it is stated here
    through complex arithmetic in fp64, independently of the real-arithmetic formulation the workloads are generated
    with.  Returns fp64."""
    batch, seq, heads, width = x.shape
    pairs = torch.view_as_complex(x.double().reshape(batch, seq, heads, width // 2, 2).contiguous())
    frequency = float(theta) ** (-2.0 * torch.arange(width // 2, dtype=torch.float64) / width)
    position = torch.arange(start, start + seq, dtype=torch.float64)
    rotation = torch.polar(torch.ones(seq, width // 2, dtype=torch.float64), position[:, None] * frequency[None, :])
    return torch.view_as_real(pairs * rotation[None, :, None, :]).reshape(batch, seq, heads, width)
