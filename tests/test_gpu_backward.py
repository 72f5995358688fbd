"""GPU parity of the recompute-based backward of the per-head MLA prefill
against the fp32 oracle (analytic formulas pinned to autograd), through the
C-ABI.  As in the reference harness (benchmarks/mla.py:68,113-117) the
backward is fed the oracle's own bf16-rounded O and fp32 LSE, so forward and
backward are tested independently."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16

pytestmark = pytest.mark.gpu


def _backward_case(cuda, batch, seq, heads, nope, rope, dv, seed, heads_checked=None, dout_factor=1.0):
    q, k, v, scale = configs.mla_prefill_inputs(batch, seq, heads, nope=nope, rope=rope, dv=dv, seed=seed,
                                                rotate=rope > 0)
    dout = configs.mla_prefill_dout(batch, seq, heads, dv, seed=seed + 100, factor=dout_factor)
    heads_checked = list(range(heads)) if heads_checked is None else heads_checked
    out_f, lse_f = oracle.causal_attention_forward(q, k, v, scale, heads=heads_checked)
    # saved tensors: bf16 O and fp32 LSE for every head (unchecked heads get zeros: their gradients are not compared)
    out = torch.zeros(batch, seq, heads, dv, dtype=torch.bfloat16)
    lse = torch.zeros(batch, heads, seq, dtype=torch.float32)
    out[:, :, heads_checked] = out_f.bfloat16()
    lse[:, heads_checked] = lse_f
    announce("mla_prefill_backward", dict(B=batch, S=seq, H=heads, dqk=nope + rope, dv=dv))
    dq, dk, dvg = ops.mla_prefill_backward(dout.to(cuda), out.to(cuda), lse.to(cuda), q.to(cuda), k.to(cuda),
                                           v.to(cuda), scale)
    torch.cuda.synchronize()
    sub = lambda t: t[:, :, heads_checked]
    eq, ek, ev = oracle.attention_backward(sub(dout), sub(out), lse[:, heads_checked], sub(q), sub(k), sub(v), scale)
    assert_close_bf16("dQ", sub(dq.cpu()), eq)
    assert_close_bf16("dK", sub(dk.cpu()), ek)
    assert_close_bf16("dV", sub(dvg.cpu()), ev)


@pytest.mark.parametrize("batch,seq,heads", [(1, 1, 1), (2, 17, 3), (1, 65, 4), (1, 128, 8), (2, 257, 4), (1, 512, 8),
                                             (1, 1000, 2)])
def test_backward_small(cuda, batch, seq, heads):
    # ragged lengths as in benchmarks/mla.py:35-39,44, per-head 192/128 geometry
    _backward_case(cuda, batch, seq, heads, 128, 64, 128, seed=21)


@pytest.mark.parametrize("dqk,dv", [(128, 128), (64, 64)])
def test_backward_square_heads(cuda, dqk, dv):
    _backward_case(cuda, 1, 320, 4, dqk, 0, dv, seed=22)


def test_backward_constant_key_gives_zero_dq(cuda):
    """With K constant along the sequence every score of a row is equal, dS sums to zero
    over the row and dQ = dS K vanishes."""
    batch, seq, heads = 1, 192, 2
    q, k, v, scale = configs.mla_prefill_inputs(batch, seq, heads, seed=23)
    k = k[:, :1].expand(batch, seq, heads, 192).contiguous()
    dout = configs.mla_prefill_dout(batch, seq, heads, 128, seed=24)
    out_f, lse = oracle.causal_attention_forward(q, k, v, scale)
    dq, dk, dvg = ops.mla_prefill_backward(dout.to(cuda), out_f.bfloat16().to(cuda), lse.to(cuda), q.to(cuda),
                                           k.to(cuda), v.to(cuda), scale)
    torch.cuda.synchronize()
    assert dq.float().abs().max().item() <= 2e-2


def test_backward_workload_3(cuda):
    """S=4096, H=128 from seed 1 (+RoPE), dO ~ N(0,1) from seed 2; saved O / LSE and expected
    gradients from the oracle on a sample of heads."""
    batch, seq, heads = 1, 4096, 128
    q, k, v, scale = configs.mla_prefill_inputs(batch, seq, heads, seed=1)
    dout = configs.mla_prefill_dout(batch, seq, heads, 128, seed=2)
    checked = [0, 17, 38, 64, 77, 90, 111, 127]
    out_f, lse_f = oracle.causal_attention_forward(q, k, v, scale, heads=checked)
    out = torch.zeros(batch, seq, heads, 128, dtype=torch.bfloat16)
    lse = torch.zeros(batch, heads, seq)
    out[:, :, checked] = out_f.bfloat16()
    lse[:, checked] = lse_f
    announce("mla_prefill_backward workload 3")
    dq, dk, dvg = ops.mla_prefill_backward(dout.to(cuda), out.to(cuda), lse.to(cuda), q.to(cuda), k.to(cuda),
                                           v.to(cuda), scale)
    torch.cuda.synchronize()
    sub = lambda t: t[:, :, checked]
    eq, ek, ev = oracle.attention_backward(sub(dout), sub(out), lse[:, checked], sub(q), sub(k), sub(v), scale)
    assert_close_bf16("dQ", sub(dq.cpu()), eq)
    assert_close_bf16("dK", sub(dk.cpu()), ek)
    assert_close_bf16("dV", sub(dvg.cpu()), ev)


# ---- absorbed backward (dscuda_mla_backward) ------------------------------------

@pytest.mark.parametrize("batch,tokens,heads", configs.MLA_TEST_PREFILL + configs.MLA_FULL_PREFILL + [(1, 96, 20), (1, 1024, 16),
                                                                                             (1, 256, 128), (2, 160, 128),
                                                                                             (1, 33, 160), (2, 50, 1),
                                                                                             # row tiles that start and end inside
                                                                                             # tokens, workgroups of one wave's rows
                                                                                             (3, 33, 7), (1, 200, 2), (2, 64, 33),
                                                                                             (1, 31, 64), (1, 97, 5), (1, 2, 48)])
def test_absorbed_backward(cuda, batch, tokens, heads):
    """Shapes of benchmarks/mla.py:34-45; dO = 0.2 * N(0,1) as at :108; saved O (bf16) and LSE
    come from the oracle forward as at :68,113-117."""
    # dLatent sums over all heads: with 128 of them dO is scaled down so that the sums stay where half a bf16 ulp
    # (the rounding of the result itself) is below the tolerance
    _absorbed_case(cuda, batch, tokens, heads, seed=77, dout_factor=0.2 if heads <= 32 else 0.05)


def _absorbed_case(cuda, batch, tokens, heads, seed, dout_factor):
    ql, qr, c, kr, scale = configs.mla_absorbed_inputs(batch, tokens, heads)
    g = torch.Generator().manual_seed(seed)
    dout = (torch.randn(batch, tokens, heads, 512, generator=g) * dout_factor).bfloat16()
    mask = oracle.causal_mask(tokens)
    out, lse = oracle.mla_forward(ql, qr, c, kr, scale, mask)
    announce("mla_backward", dict(B=batch, T=tokens, H=heads))
    grads = ops.mla_backward(dout.to(cuda), out.to(cuda), lse.to(cuda), ql.to(cuda), qr.to(cuda), c.to(cuda),
                             kr.to(cuda), scale)
    torch.cuda.synchronize()
    expected = oracle.mla_backward_unrounded(dout, out, lse, ql, qr, c, kr, scale, mask)
    for name, actual, reference in zip(("dq_latent", "dq_rope", "dlatent", "dk_rope"), grads, expected):
        assert_close_bf16(name, actual.cpu(), reference)


def test_absorbed_backward_closed_form_constant_fill(cuda):
    """benchmarks/attention/benchmark_mla.cu:38-47 with dO = 2**-6: dS == 0, so dq_latent = dq_rope =
    dk_rope = 0 and dLatent[k] = H * dO * (Harm(T) - Harm(k))."""
    batch, tokens, heads = 1, 96, 4
    ql = torch.full((batch, tokens, heads, 512), 0.125).bfloat16()
    qr = torch.full((batch, tokens, heads, 64), -0.0625).bfloat16()
    c = torch.full((batch, tokens, 512), 0.25).bfloat16()
    kr = torch.full((batch, tokens, 64), 0.03125).bfloat16()
    dout = torch.full((batch, tokens, heads, 512), 0.015625).bfloat16()
    scale = 1.0 / 24.0
    out, lse = oracle.mla_forward(ql, qr, c, kr, scale, oracle.causal_mask(tokens))
    grads = ops.mla_backward(dout.to(cuda), out.to(cuda), lse.to(cuda), ql.to(cuda), qr.to(cuda), c.to(cuda),
                             kr.to(cuda), scale)
    torch.cuda.synchronize()
    dq, dqr, dlat, dkr = (x.cpu().float() for x in grads)
    assert dq.abs().max() <= 1e-3 and dqr.abs().max() <= 1e-3 and dkr.abs().max() <= 1e-3
    harmonic = torch.cumsum(1.0 / torch.arange(1, tokens + 1, dtype=torch.float64), 0)
    before = torch.cat([torch.zeros(1, dtype=torch.float64), harmonic[:-1]])
    expected = (heads * 0.015625 * (harmonic[-1] - before)).float()
    assert (dlat - expected[None, :, None]).abs().max() <= 4e-3  # bf16 rounding of values up to 0.32


@pytest.mark.parametrize("batch,seq,heads,budget_pairs,expected_chunk", [
    (2, 640, 12, 9.5, 8),     # 24 pairs in chunks of 8 (a multiple of 8 when the budget allows one)
    (1, 640, 7, 2.5, 2),      # 7 pairs in chunks of 2, 2, 2, 1
    (1, 300, 3, 0.5, 1),      # a budget below one pair still runs, one pair at a time
])
def test_backward_in_chunks_of_pairs(cuda, batch, seq, heads, budget_pairs, expected_chunk):
    """The dS workspace is bounded: with a limit that holds only some (batch, head) pairs the two gradient passes run
    chunk after chunk over one set of dS blocks, and the workspace the library asks for shrinks accordingly."""
    key_blocks, tiles = (seq + 127) // 128, (seq + 63) // 64
    blocks = sum(tiles - 2 * kb for kb in range(key_blocks))
    limit = int(budget_pairs * blocks * 16384)
    ops.mla_prefill_backward_set_workspace_limit(limit)
    try:
        statistics = batch * heads * tiles * 128
        elements = ops.mla_prefill_backward_workspace_elements(batch, seq, heads, 192, 128)
        assert elements == statistics + expected_chunk * blocks * 4096, (elements, statistics, expected_chunk, blocks)
        assert expected_chunk * blocks * 16384 <= limit or expected_chunk == 1
        _backward_case(cuda, batch, seq, heads, 128, 64, 128, seed=31)
    finally:
        ops.mla_prefill_backward_set_workspace_limit(0)
    assert ops.mla_prefill_backward_workspace_elements(batch, seq, heads, 192, 128) == statistics + batch * heads * blocks * 4096


@pytest.mark.parametrize("batch,tokens,heads,interval_tiles", [
    (1, 256, 128, 256),   # 4 intervals, 20 items: key block 0 has four parts, the last two blocks one
    (2, 160, 128, 100),   # two batch elements, a short last interval, interval ends inside key blocks
    (1, 512, 8, 7),       # many short intervals
    (2, 257, 4, 1000),    # one interval: every key block whole
    (1, 95, 3, 4),        # 285 rows: the last half tile of 16 rows holds 13
    (1, 50, 1, 1),        # 50 rows: the last row tile holds 18, its second half tile two; one key block, cut in two
    (3, 77, 5, 3),        # 385 rows: one row in the last tile, whose second half tile is past the end
])
def test_absorbed_backward_interval_cut(cuda, batch, tokens, heads, interval_tiles):
    """The cut of the key gradients for inputs that outgrow the caches (items of one interval of row tiles and one
    key block), forced at sizes the oracle can check."""
    ops.mla_backward_set_key_interval_tiles(interval_tiles)
    try:
        _absorbed_case(cuda, batch, tokens, heads, seed=78, dout_factor=0.2 if heads <= 32 else 0.05)
    finally:
        ops.mla_backward_set_key_interval_tiles(0)


def test_absorbed_backward_interval_cut_chosen_by_the_library(cuda):
    """B=5, T=300, H=128: 38 400 rows of 2176 bytes per batch element are above the library's own bound for the
    interval cut, and on 256 compute units it cuts into intervals of 24 row tiles (725 items; the choice itself is
    pinned on the host, tests/host/index_math_test.cpp)."""
    _absorbed_case(cuda, 5, 300, 128, seed=79, dout_factor=0.05)


def test_backward_workspace_is_bounded(cuda):
    """Workload 5 (S=16384, H=128) asks for less than 4 GiB; workload 3 still fits one launch."""
    long_case = ops.mla_prefill_backward_workspace_elements(1, 16384, 128, 192, 128)
    assert long_case * 4 < 4 << 30, long_case
    tiles, key_blocks = 64, 32
    blocks = sum(tiles - 2 * kb for kb in range(key_blocks))
    assert ops.mla_prefill_backward_workspace_elements(1, 4096, 128, 192, 128) == 128 * tiles * 128 + 128 * blocks * 4096
