"""Pins of the CPU oracle: every function of ``oracle/attention_oracle.py`` is
checked against something that does not share its formula -- a library routine
(``scaled_dot_product_attention``, ``autograd``), an fp64 brute-force loop, a
closed form of the reference's constant-fill profiler inputs, or an invariant
the mathematics fixes.  A dropped term, a sign error, a transposed operand or a
wrong mask fails at least one of these."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attention_oracle as oracle


def _rand(shape, seed, factor=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float64) * factor).to(dtype)


# ---------------------------------------------------------------------------
# causal attention forward
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dqk,dv,hq,hkv", [(64, 64, 4, 4), (192, 128, 3, 3), (128, 128, 8, 2), (128, 128, 4, 1)])
def test_forward_matches_sdpa(dqk, dv, hq, hkv):
    b, s = 2, 97
    q, k, v = _rand((b, s, hq, dqk), 1), _rand((b, s, hkv, dqk), 2), _rand((b, s, hkv, dv), 3)
    scale = dqk ** -0.5
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    group = hq // hkv
    kk, vv = k.repeat_interleave(group, 2), v.repeat_interleave(group, 2)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2),
                                         is_causal=True, scale=scale).transpose(1, 2)
    assert (out - ref).abs().max() < 2e-5
    scores = torch.einsum("bqhd,bkhd->bhqk", q, kk) * scale
    scores = scores.masked_fill(~torch.ones(s, s, dtype=torch.bool).tril(), -math.inf)
    assert (lse - torch.logsumexp(scores, -1)).abs().max() < 2e-5


def test_forward_brute_force_fp64():
    """Triple loop in numpy float64, no masking tensor, no softmax routine."""
    b, s, h, dqk, dv = 1, 9, 2, 6, 5
    q, k, v = (_rand(shape, seed, dtype=torch.float64) for seed, shape in
               enumerate([(b, s, h, dqk), (b, s, h, dqk), (b, s, h, dv)], 10))
    scale = 0.37
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    qn, kn, vn = q.numpy(), k.numpy(), v.numpy()
    for hh in range(h):
        for i in range(s):
            weights = [math.exp(scale * float(np.dot(qn[0, i, hh], kn[0, j, hh]))) for j in range(i + 1)]
            total = sum(weights)
            expected = sum(w * vn[0, j, hh] for j, w in enumerate(weights)) / total
            assert np.allclose(out[0, i, hh].numpy(), expected, atol=1e-12)
            assert abs(lse[0, hh, i].item() - math.log(total)) < 1e-12


def test_forward_invariants():
    b, s, h, dqk, dv = 1, 33, 2, 192, 128
    q, k, v = _rand((b, s, h, dqk), 20, 0.5), _rand((b, s, h, dqk), 21, 0.5), _rand((b, s, h, dv), 22, 0.5)
    scale = dqk ** -0.5
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    # row 0 sees key 0 only
    assert torch.allclose(out[:, 0], v[:, 0], atol=1e-6)
    assert torch.allclose(lse[:, :, 0], (q[:, 0] * k[:, 0]).sum(-1) * scale, atol=1e-5)
    # adding a constant c to every score (extra dimension with q=1, k=c/scale) shifts LSE by c, keeps O
    shift = 0.75
    q2 = torch.cat([q, torch.ones(b, s, h, 1)], -1)
    k2 = torch.cat([k, torch.full((b, s, h, 1), shift / scale)], -1)
    out2, lse2 = oracle.causal_attention_forward(q2, k2, v, scale)
    assert torch.allclose(out2, out, atol=1e-5)
    assert torch.allclose(lse2, lse + shift, atol=1e-5)
    # constant V passes through untouched (probabilities sum to one)
    out3, _ = oracle.causal_attention_forward(q, k, torch.full_like(v, 0.3), scale)
    assert torch.allclose(out3, torch.full_like(out3, 0.3), atol=1e-6)
    # the head subset selects, it does not change values
    sub, sub_lse = oracle.causal_attention_forward(q, k, v, scale, heads=[1])
    assert torch.equal(sub[:, :, 0], out[:, :, 1]) and torch.equal(sub_lse[:, 0], lse[:, 1])


# ---------------------------------------------------------------------------
# attention backward
# ---------------------------------------------------------------------------

def _autograd_reference(q, k, v, dout, scale):
    q, k, v = (x.clone().requires_grad_() for x in (q, k, v))
    s = q.shape[1]
    scores = torch.einsum("bqhd,bkhd->bhqk", q, k) * scale
    scores = scores.masked_fill(~torch.ones(s, s, dtype=torch.bool).tril(), -math.inf)
    out = torch.einsum("bhqk,bkhd->bqhd", scores.softmax(-1), v)
    return torch.autograd.grad(out, (q, k, v), dout)


@pytest.mark.parametrize("dqk,dv", [(192, 128), (64, 64)])
def test_backward_matches_autograd(dqk, dv):
    b, s, h = 2, 41, 3
    q, k, v = (_rand(shape, seed, 0.5, torch.float64) for seed, shape in
               enumerate([(b, s, h, dqk), (b, s, h, dqk), (b, s, h, dv)], 30))
    dout = _rand((b, s, h, dv), 33, 1.0, torch.float64)
    scale = dqk ** -0.5
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    dq, dk, dv_ = oracle.attention_backward(dout, out, lse, q, k, v, scale)
    rq, rk, rv = _autograd_reference(q, k, v, dout, scale)
    for name, a, r in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv_, rv)):
        assert (a - r).abs().max() < 1e-10, name


@pytest.mark.parametrize("q_heads,kv_heads", [(4, 2), (8, 1), (6, 3)])
def test_grouped_query_backward_matches_autograd(q_heads, kv_heads):
    """dK and dV of a shared key/value head are the sums over the query heads that read it: autograd through an
    explicit repeat_interleave of K and V (the reference's own GQA formulation, benchmarks/flash_attention.py:72-74)
    says so, and a wrong head mapping (h % Hkv instead of h // group) or a missing term fails it."""
    b, s, d = 2, 29, 16
    q = _rand((b, s, q_heads, d), 50, 0.5, torch.float64).requires_grad_()
    k = _rand((b, s, kv_heads, d), 51, 0.5, torch.float64).requires_grad_()
    v = _rand((b, s, kv_heads, d), 52, 0.5, torch.float64).requires_grad_()
    dout = _rand((b, s, q_heads, d), 53, 1.0, torch.float64)
    scale = d ** -0.5
    group = q_heads // kv_heads
    mask = torch.ones(s, s, dtype=torch.bool).tril()
    scores = torch.einsum("bqhd,bkhd->bhqk", q, k.repeat_interleave(group, dim=2)) * scale
    out = torch.einsum("bhqk,bkhd->bqhd", scores.masked_fill(~mask, -math.inf).softmax(-1), v.repeat_interleave(group, dim=2))
    rq, rk, rv = torch.autograd.grad(out, (q, k, v), dout)
    saved, lse = oracle.causal_attention_forward(q.detach(), k.detach(), v.detach(), scale)
    assert (saved - out.detach()).abs().max() < 1e-12
    dq, dk, dv = oracle.attention_backward(dout, saved, lse, q.detach(), k.detach(), v.detach(), scale)
    assert dk.shape == k.shape and dv.shape == v.shape
    for name, a, r in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        assert (a - r).abs().max() < 1e-10, name


def test_backward_finite_differences():
    b, s, h, dqk, dv = 1, 7, 1, 4, 3
    q, k, v = (_rand(shape, seed, 1.0, torch.float64) for seed, shape in
               enumerate([(b, s, h, dqk), (b, s, h, dqk), (b, s, h, dv)], 40))
    dout = _rand((b, s, h, dv), 43, 1.0, torch.float64)
    scale = 0.6
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    grads = oracle.attention_backward(dout, out, lse, q, k, v, scale)

    def loss(qq, kk, vv):
        return (oracle.causal_attention_forward(qq, kk, vv, scale)[0] * dout).sum().item()

    eps = 1e-6
    for index, (tensor, grad) in enumerate(zip((q, k, v), grads)):
        flat = tensor.reshape(-1)
        for position in range(0, flat.numel(), 3):
            plus, minus = tensor.clone(), tensor.clone()
            plus.reshape(-1)[position] += eps
            minus.reshape(-1)[position] -= eps
            args_p = [q, k, v]
            args_m = [q, k, v]
            args_p[index], args_m[index] = plus, minus
            numeric = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(numeric - grad.reshape(-1)[position].item()) < 1e-6


def test_backward_row_sum_of_dscore_is_zero():
    """sum_k dS[q,k] = 0  <=>  dQ is orthogonal to nothing in particular but
    dS K summed against a constant key gives zero: with K constant along the
    sequence, dQ must vanish."""
    b, s, h, dqk, dv = 1, 19, 2, 16, 8
    q = _rand((b, s, h, dqk), 50, 1.0, torch.float64)
    k = _rand((b, 1, h, dqk), 51, 1.0, torch.float64).expand(b, s, h, dqk).contiguous()
    v = _rand((b, s, h, dv), 52, 1.0, torch.float64)
    dout = _rand((b, s, h, dv), 53, 1.0, torch.float64)
    out, lse = oracle.causal_attention_forward(q, k, v, 0.25)
    dq, _, _ = oracle.attention_backward(dout, out, lse, q, k, v, 0.25)
    assert dq.abs().max() < 1e-12


# ---------------------------------------------------------------------------
# absorbed MLA
# ---------------------------------------------------------------------------

def test_mla_forward_is_mqa_over_concatenated_heads():
    b, t, h = 2, 37, 5
    ql, qr = _rand((b, t, h, 512), 60, 0.25), _rand((b, t, h, 64), 61, 0.25)
    c, kr = _rand((b, t, 512), 62, 0.25), _rand((b, t, 64), 63, 0.25)
    scale = 576 ** -0.5
    out, lse = oracle.mla_forward_unrounded(ql, qr, c, kr, scale, oracle.causal_mask(t))
    q = torch.cat([ql, qr], -1)
    k = torch.cat([c, kr], -1)[:, :, None]
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2).expand(b, h, t, 576),
                                         c[:, None].expand(b, h, t, 512), is_causal=True, scale=scale)
    assert (out - ref.transpose(1, 2)).abs().max() < 2e-5
    # and equals the per-head oracle fed with the broadcast KV head
    out2, lse2 = oracle.causal_attention_forward(q, k, c[:, :, None], scale)
    assert (out - out2).abs().max() < 2e-5 and (lse - lse2).abs().max() < 2e-5
    rounded, lse3 = oracle.mla_forward(ql, qr, c, kr, scale, oracle.causal_mask(t))
    assert rounded.dtype == torch.bfloat16 and torch.equal(rounded, out.bfloat16()) and torch.equal(lse3, lse)


def test_mla_constant_fill_closed_form():
    """Constants of benchmarks/attention/benchmark_mla.cu:38-47 (q_lat=1/8, q_rope=-1/16, c=1/4,
    k_rope=1/32, dO=1/64, scale=1/24): every score is (16-0.125)/24, O == 0.25,
    LSE[t] = score + ln(t+1); dP == delta so dS == 0 and only the value path
    feeds dLatent: dLatent[k] = H * dO * (Harm(T) - Harm(k))."""
    b, t, h = 1, 24, 3
    ql = torch.full((b, t, h, 512), 0.125)
    qr = torch.full((b, t, h, 64), -0.0625)
    c = torch.full((b, t, 512), 0.25)
    kr = torch.full((b, t, 64), 0.03125)
    scale = 1.0 / 24.0
    mask = oracle.causal_mask(t)
    out, lse = oracle.mla_forward_unrounded(ql, qr, c, kr, scale, mask)
    score = (512 * 0.125 * 0.25 - 64 * 0.0625 * 0.03125) / 24
    assert abs(score - 0.6614583333) < 1e-9
    assert torch.allclose(out, torch.full_like(out, 0.25), atol=1e-6)
    expected_lse = score + torch.log(torch.arange(1, t + 1, dtype=torch.float32))
    assert torch.allclose(lse, expected_lse[None, None].expand(b, h, t), atol=1e-5)
    dout = torch.full((b, t, h, 512), 0.015625)
    dq, dqr, dlat, dkr = oracle.mla_backward_unrounded(dout, out, lse, ql, qr, c, kr, scale, mask)
    assert dq.abs().max() < 1e-6 and dqr.abs().max() < 1e-6 and dkr.abs().max() < 1e-6
    harmonic = torch.cumsum(1.0 / torch.arange(1, t + 1, dtype=torch.float64), 0)
    harm_before = torch.cat([torch.zeros(1, dtype=torch.float64), harmonic[:-1]])
    expected = (h * 0.015625 * (harmonic[-1] - harm_before)).float()
    assert torch.allclose(dlat, expected[None, :, None].expand(b, t, 512), atol=1e-5)


def test_mla_backward_matches_autograd():
    """The way the reference builds its expected gradients (benchmarks/mla.py:108-110)."""
    b, t, h = 2, 17, 3
    tensors = [_rand(shape, seed, 0.25, torch.float64) for seed, shape in
               enumerate([(b, t, h, 512), (b, t, h, 64), (b, t, 512), (b, t, 64)], 70)]
    dout = _rand((b, t, h, 512), 74, 0.2, torch.float64)
    scale = 576 ** -0.5
    mask = oracle.causal_mask(t)
    leaves = [x.clone().requires_grad_() for x in tensors]
    out, lse = oracle.mla_forward_unrounded(*leaves, scale, mask)
    expected = torch.autograd.grad(out, leaves, dout)
    actual = oracle.mla_backward_unrounded(dout, out.detach(), lse.detach(), *tensors, scale, mask)
    for a, e in zip(actual, expected):
        assert (a - e).abs().max() < 1e-10
    rounded = oracle.mla_backward(dout, out.detach(), lse.detach(), *tensors, scale, mask)
    assert all(r.dtype == torch.bfloat16 for r in rounded)


# ---------------------------------------------------------------------------
# decode
# ---------------------------------------------------------------------------

def test_decode_matches_sdpa_with_length_mask():
    b, n, h = 3, 70, 4
    q = _rand((b, 1, h, 576), 80, 0.5)
    cache = _rand((b, n, 576), 81, 0.5)
    lengths = torch.tensor([1, 33, 70])
    scale = 192 ** -0.5
    out, lse = oracle.mla_decode_unrounded(q, cache, lengths, scale)
    assert out.shape == (b, 1, h, 512) and lse.shape == (b, h, 1)
    for i in range(b):
        ln = int(lengths[i])
        keys = cache[i, :ln][None, None].expand(1, h, ln, 576)
        ref = F.scaled_dot_product_attention(q[i].transpose(0, 1)[None], keys, keys[..., :512], scale=scale)
        assert (out[i, 0] - ref[0, :, 0]).abs().max() < 2e-5
        scores = torch.einsum("hd,kd->hk", q[i, 0], cache[i, :ln]) * scale
        assert (lse[i, :, 0] - torch.logsumexp(scores, -1)).abs().max() < 2e-5


def test_decode_full_length_equals_last_prefill_row():
    b, t, h = 2, 29, 3
    ql, qr = _rand((b, t, h, 512), 90, 0.25), _rand((b, t, h, 64), 91, 0.25)
    c, kr = _rand((b, t, 512), 92, 0.25), _rand((b, t, 64), 93, 0.25)
    scale = 576 ** -0.5
    out, lse = oracle.mla_forward_unrounded(ql, qr, c, kr, scale, oracle.causal_mask(t))
    packed_q = torch.cat([ql[:, -1:], qr[:, -1:]], -1)
    dec, dec_lse = oracle.mla_decode_unrounded(packed_q, torch.cat([c, kr], -1), torch.tensor([t, t]), scale)
    assert (dec[:, 0] - out[:, -1]).abs().max() < 1e-5 and (dec_lse[:, :, 0] - lse[:, :, -1]).abs().max() < 1e-5


def test_decode_constant_fill_closed_form():
    """benchmarks/attention/benchmark_mla_decode.cu:42-48: q = 1/8, cache = 1/4,
    scale = 1/24 -> score 0.75, O == 0.25, LSE = 0.75 + ln(context)."""
    b, n, h = 2, 100, 4
    q = torch.full((b, 1, h, 576), 0.125)
    cache = torch.full((b, n, 576), 0.25)
    lengths = torch.tensor([100, 37])
    out, lse = oracle.mla_decode_unrounded(q, cache, lengths, 1.0 / 24.0)
    assert torch.allclose(out, torch.full_like(out, 0.25), atol=1e-6)
    expected = 0.75 + torch.log(lengths.float())
    assert torch.allclose(lse[:, :, 0], expected[:, None].expand(b, h), atol=1e-5)


# ---------------------------------------------------------------------------
# page packing, workspace size
# ---------------------------------------------------------------------------

def test_pack_cache_closed_form():
    kv = _rand((3, 130, 576), 100).bfloat16()
    paged, table = oracle.pack_cache(kv, 64)
    assert paged.shape == (9, 64, 1, 576) and table.dtype == torch.int32
    assert torch.equal(table, torch.arange(9, dtype=torch.int32).reshape(3, 3))
    for bi in range(3):
        for token in (0, 63, 64, 129):
            assert torch.equal(paged[table[bi, token // 64], token % 64, 0], kv[bi, token])
        assert paged[table[bi, 2], 2:].abs().max() == 0  # padding is zero


def test_workspace_elements():
    assert oracle.decode_workspace_elements(2, 3, 8, 512) == 2 * 3 * 8 * 514
    assert oracle.decode_workspace_elements(64, 128, 8, 512) == 64 * 128 * 8 * 514


def test_projections_brute_force_and_absorption_identity():
    """absorb_query / unabsorb_output against explicit loops in fp64, and the identity that makes absorption valid:
    per-head attention with k_nope = latent W_UK^T and v = latent W_UV^T gives the same output as absorbed attention
    over the latent itself between the two projections."""
    g = torch.Generator().manual_seed(11)
    tokens, heads, d, c = 5, 3, 128, 512
    q_nope = torch.randn(tokens, heads, d, generator=g, dtype=torch.float64)
    w_uk = torch.randn(heads, d, c, generator=g, dtype=torch.float64) * 0.05
    w_uv = torch.randn(heads, d, c, generator=g, dtype=torch.float64) * 0.05
    latent = torch.randn(tokens, c, generator=g, dtype=torch.float64)
    q_latent = oracle.absorb_query(q_nope.float(), w_uk.float()).double()
    for t_index in (0, 4):
        for h in range(heads):
            for col in (0, 77, 511):
                expected = sum(q_nope[t_index, h, k] * w_uk[h, k, col] for k in range(d))
                assert abs(q_latent[t_index, h, col] - expected) < 1e-4
    o_latent = torch.randn(tokens, heads, c, generator=g, dtype=torch.float64)
    out = oracle.unabsorb_output(o_latent.float(), w_uv.float()).double()
    for t_index in (1, 3):
        for h in range(heads):
            for col in (0, 64, 127):
                expected = sum(o_latent[t_index, h, k] * w_uv[h, col, k] for k in range(c))
                assert abs(out[t_index, h, col] - expected) < 1e-3
    # the identity, in fp64 through the same functions
    q_abs = oracle.absorb_query(q_nope, w_uk)                        # [T, H, C]
    scale = 0.1
    mask = oracle.causal_mask(tokens)
    scores_absorbed = torch.einsum("thc,sc->hts", q_abs, latent) * scale
    k_nope = torch.einsum("sc,hdc->shd", latent, w_uk)               # [S, H, D]
    scores_heads = torch.einsum("thd,shd->hts", q_nope, k_nope) * scale
    assert (scores_absorbed - scores_heads).abs().max() < 1e-9
    p = torch.softmax(scores_heads.masked_fill(~mask, float("-inf")), dim=-1)
    v = torch.einsum("sc,hdc->shd", latent, w_uv)
    out_heads = torch.einsum("hts,shd->thd", p, v)
    out_absorbed = oracle.unabsorb_output(torch.einsum("hts,sc->thc", p, latent), w_uv)
    assert (out_heads - out_absorbed).abs().max() < 1e-9


# ---- rotary embedding ----------------------------------------------------------------------------------------

def _rope_variant(x, theta, pairing="interleaved", direction=1.0, exponent=2.0):
    """Real-arithmetic RoPE with one knob per plausible mistake: how columns pair up, which way the pair turns,
    and the frequency exponent."""
    _, seq, _, width = x.shape
    half = width // 2
    frequency = theta ** (-exponent * torch.arange(half, dtype=torch.float64) / width)
    angle = direction * torch.arange(seq, dtype=torch.float64)[:, None] * frequency[None]
    cos, sin = angle.cos()[None, :, None], angle.sin()[None, :, None]
    x = x.double()
    out = torch.empty_like(x)
    if pairing == "interleaved":
        a, b = x[..., 0::2], x[..., 1::2]
        out[..., 0::2], out[..., 1::2] = a * cos - b * sin, a * sin + b * cos
    else:   # first half with second half
        a, b = x[..., :half], x[..., half:]
        out[..., :half], out[..., half:] = a * cos - b * sin, a * sin + b * cos
    return out


def test_rope_closed_forms():
    theta, width, seq = 10000.0, 64, 300
    # (1, 0) in every pair at position p -> (cos, sin) of p * theta^(-2i/R), written out with math.cos / math.sin
    unit = torch.zeros(1, seq, 1, width)
    unit[..., 0::2] = 1.0
    rotated = oracle.apply_rope(unit, theta)
    for p in (0, 1, 7, 299):
        for i in (0, 1, 5, 31):
            angle = p * theta ** (-2.0 * i / width)
            assert abs(rotated[0, p, 0, 2 * i].item() - math.cos(angle)) < 1e-12
            assert abs(rotated[0, p, 0, 2 * i + 1].item() - math.sin(angle)) < 1e-12
    # (0, 1) -> (-sin, cos): the pair turns counter-clockwise
    unit = torch.zeros(1, seq, 1, width)
    unit[..., 1::2] = 1.0
    rotated = oracle.apply_rope(unit, theta)
    angle = 7 * theta ** (-2.0 * 5 / width)
    assert abs(rotated[0, 7, 0, 10].item() + math.sin(angle)) < 1e-12 and abs(rotated[0, 7, 0, 11].item() - math.cos(angle)) < 1e-12
    # position 0 is the identity; R = 2 leaves one pair turning by exactly p radians whatever theta is
    x = torch.randn(2, 5, 3, width, generator=torch.Generator().manual_seed(5), dtype=torch.float64)
    assert torch.equal(oracle.apply_rope(x, theta)[:, 0], x[:, 0])
    pair = torch.tensor([0.3, -1.1], dtype=torch.float64).expand(1, 9, 1, 2)
    for any_theta in (10000.0, 3.0):
        turned = oracle.apply_rope(pair, any_theta)
        for p in range(9):
            assert abs(turned[0, p, 0, 0].item() - (0.3 * math.cos(p) + 1.1 * math.sin(p))) < 1e-12
            assert abs(turned[0, p, 0, 1].item() - (0.3 * math.sin(p) - 1.1 * math.cos(p))) < 1e-12


def test_rope_composes_and_depends_on_relative_position_only():
    theta, width = 10000.0, 64
    g = torch.Generator().manual_seed(6)
    q = torch.randn(1, 40, 2, width, generator=g, dtype=torch.float64)
    k = torch.randn(1, 40, 2, width, generator=g, dtype=torch.float64)
    # start position s: the same as rotating a longer run and taking its tail
    shifted = oracle.apply_rope(q, theta, start=11)
    padded = torch.cat([torch.zeros(1, 11, 2, width, dtype=torch.float64), q], 1)
    torch.testing.assert_close(shifted, oracle.apply_rope(padded, theta)[:, 11:], atol=1e-12, rtol=0)
    # <rope(q, m), rope(k, n)> depends on m - n only
    rq, rk = oracle.apply_rope(q, theta), oracle.apply_rope(k, theta)
    rq5, rk5 = oracle.apply_rope(q, theta, start=5), oracle.apply_rope(k, theta, start=5)
    torch.testing.assert_close(torch.einsum("bmhd,bnhd->bhmn", rq, rk), torch.einsum("bmhd,bnhd->bhmn", rq5, rk5),
                               atol=1e-10, rtol=0)


def test_rope_workload_formulation_matches_the_oracle_and_mistakes_do_not():
    from dscuda_amd.harness import configs
    theta, width = 10000.0, 64
    x = torch.randn(2, 257, 3, width, generator=torch.Generator().manual_seed(7)) * 0.5
    expected = oracle.apply_rope(x, theta)
    # the formulation every workload is generated with (fp32 sine / cosine, fp32 products)
    torch.testing.assert_close(configs.apply_rope(x, theta).double(), expected, atol=2e-6, rtol=0)
    torch.testing.assert_close(_rope_variant(x, theta), expected, atol=1e-12, rtol=0)
    # each plausible mistake is far outside that
    for mistake in (dict(pairing="halves"), dict(direction=-1.0), dict(exponent=1.0)):
        assert (_rope_variant(x, theta, **mistake) - expected).abs().max() > 0.1, mistake
