"""GPU parity of the absorbed MLA decode (paged latent cache, split-KV) and of
the absorbed causal prefill forward against the fp32 oracle, through the C-ABI."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16, assert_close_lse

pytestmark = pytest.mark.gpu


def _decode_case(cuda, batch, tokens, heads, lengths, splits=8, page_size=64, seed=2026, factor=0.25,
                 permute_pages=False, scale=None):
    g = torch.Generator().manual_seed(seed)
    query = (torch.randn(batch, 1, heads, 576, generator=g) * factor).bfloat16()
    cache = (torch.randn(batch, tokens, 576, generator=g) * factor).bfloat16()
    scale = configs.c_float(576 ** -0.5) if scale is None else scale
    paged, table = configs.pack_cache(cache, page_size)
    if permute_pages:
        order = torch.randperm(paged.shape[0], generator=g)
        inverse = torch.empty_like(order)
        inverse[order] = torch.arange(order.numel())
        paged = paged[order].contiguous()      # new block i holds old block order[i]
        table = inverse[table.long()].to(torch.int32)
    lengths_t = torch.tensor(lengths, dtype=torch.int32)
    announce("mla_decode", dict(B=batch, KV=tokens, H=heads, lengths=lengths, splits=splits, page=page_size,
                                permuted=permute_pages))
    out, lse = ops.mla_decode(query.to(cuda), paged.to(cuda), table.to(cuda), lengths_t.to(cuda), scale,
                              splits=splits)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.mla_decode_unrounded(query, cache, lengths_t, scale)
    assert_close_bf16("O", out, expected)
    assert_close_lse("LSE", lse, expected_lse)
    return out, lse


@pytest.mark.parametrize("batch,tokens,heads", configs.MLA_TEST_DECODE)
def test_decode_reference_test_shapes(cuda, batch, tokens, heads):
    # benchmarks/mla.py:36-39 with the test-mode lengths (1, ..., T) of :58-61
    _decode_case(cuda, batch, tokens, heads, configs.harness_decode_lengths(batch, tokens, test=True))


@pytest.mark.parametrize("batch,tokens,heads", [(2, 1024, 16), (1, 256, 16), (4, 4096, 32), (4, 4096, 128)])
def test_decode_reference_benchmark_shapes(cuda, batch, tokens, heads):
    _decode_case(cuda, batch, tokens, heads, configs.harness_decode_lengths(batch, tokens, test=False))


@pytest.mark.parametrize("splits", [1, 2, 3, 8, 32])
def test_decode_is_split_invariant(cuda, splits):
    _decode_case(cuda, 5, 700, 128, [1, 63, 64, 65, 700], splits=splits, seed=7)


@pytest.mark.parametrize("batch,splits", [(1, 2), (1, 3), (2, 2), (1, 8)])
def test_decode_small_batches_keep_inside_the_workspace(cuda, batch, splits):
    """batch * (splits - 1) < 3: the cases in which slots plus flag words come closest to the end of the
    workspace.  The workspace is followed by a guard region that must come back untouched."""
    heads, tokens = 128, 700
    g = torch.Generator().manual_seed(70 + batch + splits)
    query = (torch.randn(batch, 1, heads, 576, generator=g) * 0.25).bfloat16()
    cache = (torch.randn(batch, tokens, 576, generator=g) * 0.25).bfloat16()
    lengths = torch.tensor([tokens - 37 * b for b in range(batch)], dtype=torch.int32)
    scale = configs.c_float(576 ** -0.5)
    paged, table = configs.pack_cache(cache, 64)
    elements = ops.mla_library().workspace(batch, heads, splits, 512)
    guard = 4096
    buffer = torch.full((elements + guard,), 12345.0, device=cuda, dtype=torch.float32)
    announce("mla_decode guard", dict(B=batch, splits=splits, workspace_elements=elements))
    out, lse = ops.mla_decode(query.to(cuda), paged.to(cuda), table.to(cuda), lengths.to(cuda), scale, splits=splits,
                              workspace=buffer[:elements])
    torch.cuda.synchronize()
    assert torch.equal(buffer[elements:].cpu(), torch.full((guard,), 12345.0)), "wrote past the workspace"
    expected, expected_lse = oracle.mla_decode_unrounded(query, cache, lengths, scale)
    assert_close_bf16("O", out, expected)
    assert_close_lse("LSE", lse, expected_lse)


def test_decode_permuted_block_table(cuda):
    _decode_case(cuda, 3, 333, 64, [333, 17, 200], permute_pages=True, seed=8)


@pytest.mark.parametrize("page_size", [16, 48, 128])
def test_decode_other_page_sizes(cuda, page_size):
    _decode_case(cuda, 3, 300, 32, [300, 1, 129], page_size=page_size, seed=9)


def test_decode_many_heads(cuda):
    _decode_case(cuda, 2, 200, 160, [200, 77], seed=10)


@pytest.mark.parametrize("splits,tokens,lengths,hot", [
    (1, 300, [300, 250], [(200, 260, 4.0)]),
    (8, 1500, [1500, 1250], [(1000, 1100, 4.0)]),
    (8, 1500, [1500, 1250], [(600, 650, 1.0), (1000, 1100, 4.0)]),   # the reference is raised twice in one walk
    (1, 700, [700, 433], [(45, 50, 0.5), (300, 301, 2.0), (690, 700, 8.0)]),   # in the middle of units, thrice
])
def test_decode_large_scores_raise_the_reference(cuda, splits, tokens, lengths, hot):
    """Scores that outgrow the maximum of the first keys by far more than the head room the fixed softmax
    reference leaves (2^120): late keys are aligned with the query, early ones are not.  The walk that meets
    them raises the reference of the rows concerned and scales what they had accumulated; in the cut cases
    several workgroups share the tiles of the two sequences and the parts merge as usual."""
    batch, heads = 2, 8
    g = torch.Generator().manual_seed(12)
    query = (torch.randn(batch, 1, heads, 576, generator=g)).bfloat16()
    cache = (torch.randn(batch, tokens, 576, generator=g) * 0.05).bfloat16()
    for first, last, factor in hot:   # huge positive scores late in the stream
        cache[:, first:last] = (query[:, 0, :1].float() * factor).bfloat16()
    lengths = torch.tensor(lengths, dtype=torch.int32)
    paged, table = configs.pack_cache(cache, 64)
    scale = 1.0
    announce("mla_decode raised reference", dict(splits=splits, hot=hot))
    out, lse = ops.mla_decode(query.to(cuda), paged.to(cuda), table.to(cuda), lengths.to(cuda), scale, splits=splits)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.mla_decode_unrounded(query, cache, lengths, scale)
    assert expected_lse.max() > 500  # really is far outside the fast path's range
    # outputs reach |O| ~ 15 here, where bf16 is spaced 0.06 apart: the reference harness's own relative bar
    # (benchmarks/mla.py:103-105) instead of the absolute one
    torch.testing.assert_close(out.cpu().float(), expected, atol=8e-3, rtol=8e-3)
    assert_close_bf16("O", out, expected, max_abs=1.5e-1, mean_abs=6e-3)
    worst = ((lse.cpu() - expected_lse).abs() / expected_lse.abs().clamp_min(1)).max().item()
    assert worst <= 1e-5


def test_decode_with_a_reused_plan_equals_the_plain_call(cuda):
    """One plan, several calls (the layers of a model share the cache lengths): bit-equal to the call that
    builds its own plan, also after a call over other data in between and with the workspace overwritten."""
    data = configs.mla_decode_inputs(batch=9, heads=128, low=40, high=2600, seed=41)
    on_gpu = [data[k].to(cuda) for k in ("query", "paged", "table", "lengths")]
    announce("mla_decode planned", dict(lengths=data["lengths"].tolist()))
    for splits in (8, 1):
        expected, expected_lse = ops.mla_decode(*on_gpu, data["scale"], splits=splits)
        plan = ops.mla_decode_plan(on_gpu[3], 128, splits)
        workspace = ops.mla_decode_workspace(9, 128, splits, 512, cuda)
        other_query = (on_gpu[0].float() * -0.5).bfloat16()
        for layer in range(3):
            workspace.fill_(float("nan"))
            query = on_gpu[0] if layer != 1 else other_query
            out, lse = ops.mla_decode_planned(query, on_gpu[1], on_gpu[2], on_gpu[3], plan, data["scale"], splits=splits,
                                              workspace=workspace)
            torch.cuda.synchronize()
            if layer != 1:
                assert torch.equal(out, expected) and torch.equal(lse, expected_lse)
    oracle_out, oracle_lse = oracle.mla_decode_unrounded(data["query"], data["cache"], data["lengths"], data["scale"])
    assert_close_bf16("O", expected, oracle_out)
    assert_close_lse("LSE", expected_lse, oracle_lse)


def test_decode_plan_is_read_only(cuda):
    """A plan is not written by the calls that use it, whatever their data (also data that makes rows outrun their
    softmax reference): the next call over the same plan with ordinary data gives the ordinary result."""
    batch, tokens, heads = 2, 1500, 8
    g = torch.Generator().manual_seed(43)
    query = torch.randn(batch, 1, heads, 576, generator=g).bfloat16()
    cache = (torch.randn(batch, tokens, 576, generator=g) * 0.05).bfloat16()
    hot = cache.clone()
    hot[:, 1000:1100] = (query[:, 0, :1].float() * 4.0).bfloat16()
    lengths = torch.tensor([1500, 1250], dtype=torch.int32)
    paged, table = configs.pack_cache(cache, 64)
    hot_paged, _ = configs.pack_cache(hot, 64)
    plan = ops.mla_decode_plan(lengths.to(cuda), heads, 8)
    torch.cuda.synchronize()
    before = plan.clone()
    announce("mla_decode plan reuse")
    ops.mla_decode_planned(query.to(cuda), hot_paged.to(cuda), table.to(cuda), lengths.to(cuda), plan, 1.0, splits=8)
    out, lse = ops.mla_decode_planned(query.to(cuda), paged.to(cuda), table.to(cuda), lengths.to(cuda), plan, 1.0, splits=8)
    torch.cuda.synchronize()
    assert torch.equal(plan, before)
    expected, expected_lse = oracle.mla_decode_unrounded(query, cache, lengths, 1.0)
    assert_close_bf16("O", out, expected)
    assert_close_lse("LSE", lse, expected_lse)


def test_decode_repeated_calls_never_see_stale_parts(cuda):
    """Parts of a sequence pass from workgroup to workgroup through the workspace inside one launch.  Sixty calls
    that alternate between two data sets over one workspace must each reproduce their own first result bit for
    bit: a part or a statistic left over from the other data set would show."""
    first = configs.mla_decode_inputs(batch=24, heads=128, low=300, high=5000, seed=51)
    second = configs.mla_decode_inputs(batch=24, heads=128, low=300, high=5000, seed=52)
    pages = max(first["table"].shape[1], second["table"].shape[1])
    workspace = ops.mla_decode_workspace(24, 128, 8, 512, cuda)
    sets = []
    for data in (first, second):
        table = torch.zeros(24, pages, dtype=torch.int32)
        table[:, :data["table"].shape[1]] = data["table"]
        sets.append([data["query"].to(cuda), data["paged"].to(cuda), table.to(cuda), data["lengths"].to(cuda)])
    announce("mla_decode repeated calls")
    expected = []
    for tensors, data in zip(sets, (first, second)):
        out, lse = ops.mla_decode(*tensors, data["scale"], splits=8, workspace=workspace)
        torch.cuda.synchronize()
        oracle_out, oracle_lse = oracle.mla_decode_unrounded(data["query"], data["cache"], data["lengths"], data["scale"])
        assert_close_bf16("O", out, oracle_out)
        assert_close_lse("LSE", lse, oracle_lse)
        expected.append((out.clone(), lse.clone()))
    results = []
    for call in range(60):
        which = call % 2
        out, lse = ops.mla_decode(*sets[which], first["scale"], splits=8, workspace=workspace)
        results.append((which, out, lse))
    torch.cuda.synchronize()
    for call, (which, out, lse) in enumerate(results):
        assert torch.equal(out, expected[which][0]) and torch.equal(lse, expected[which][1]), f"call {call}"


def test_decode_large_batch(cuda):
    """More sequences than any table a workgroup could hold in LDS: the plan lives in memory."""
    batch, tokens, heads = 3500, 70, 4
    lengths = [1 + (7 * b) % tokens for b in range(batch)]
    _decode_case(cuda, batch, tokens, heads, lengths, splits=2, seed=44)


def test_decode_closed_form_constant_fill(cuda):
    """benchmarks/attention/benchmark_mla_decode.cu:42-48: O == 0.25, LSE = 0.75 + ln(context)."""
    batch, context, heads = 2, 1024, 16
    query = torch.full((batch, 1, heads, 576), 0.125).bfloat16()
    cache = torch.full((batch, context, 576), 0.25).bfloat16()
    paged, table = configs.pack_cache(cache, 64)
    lengths = torch.full((batch,), context, dtype=torch.int32)
    out, lse = ops.mla_decode(query.to(cuda), paged.to(cuda), table.to(cuda), lengths.to(cuda), 1.0 / 24.0)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().float(), torch.full((batch, 1, heads, 512), 0.25))
    assert (lse.cpu() - (0.75 + torch.log(torch.tensor(float(context))))).abs().max() <= 1e-4


def test_decode_workload_4(cuda):
    """B=64, H=128, lengths ~ U[1024, 8192] from seed 3: every sequence against the oracle."""
    data = configs.mla_decode_inputs()
    lengths = data["lengths"]
    announce("mla_decode workload 4", dict(total_tokens=int(lengths.sum())))
    out, lse = ops.mla_decode(data["query"].to(cuda), data["paged"].to(cuda), data["table"].to(cuda),
                              lengths.to(cuda), data["scale"], splits=8)
    torch.cuda.synchronize()
    out, lse = out.cpu(), lse.cpu()
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    for b in range(lengths.numel()):
        n = int(lengths[b])
        expected, expected_lse = oracle.mla_decode_unrounded(
            data["query"][b:b + 1], data["cache"][b:b + 1, :n], lengths[b:b + 1], data["scale"])
        assert_close_bf16(f"O[{b}]", out[b:b + 1], expected)
        assert_close_lse(f"LSE[{b}]", lse[b:b + 1], expected_lse)


# ---- absorbed causal prefill forward (dscuda_mla_forward) ----------------------

@pytest.mark.parametrize("batch,tokens,heads", configs.MLA_TEST_PREFILL + configs.MLA_FULL_PREFILL +
                         [(1, 200, 128), (1, 1024, 16), (1, 33, 160), (2, 50, 1), (1, 70, 100)])
def test_absorbed_forward(cuda, batch, tokens, heads):
    ql, qr, c, kr, scale = configs.mla_absorbed_inputs(batch, tokens, heads)
    announce("mla_forward", dict(B=batch, T=tokens, H=heads))
    out, lse = ops.mla_forward(ql.to(cuda), qr.to(cuda), c.to(cuda), kr.to(cuda), scale)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.mla_forward_unrounded(ql, qr, c, kr, scale, oracle.causal_mask(tokens))
    assert_close_bf16("O", out, expected)
    assert_close_lse("LSE", lse, expected_lse)


def test_absorbed_forward_large_scores_raise_the_reference(cuda):
    """The prefill form of the same walk: late keys aligned with the queries give scores far above what the first
    keys gave, rows of one workgroup see different numbers of keys, and the rows that meet the hot keys raise
    their softmax reference while the others (earlier tokens) never see them."""
    batch, tokens, heads = 1, 300, 8
    g = torch.Generator().manual_seed(14)
    direction = torch.randn(576, generator=g)
    query = (direction[None, None, None, :] + 0.1 * torch.randn(batch, tokens, heads, 576, generator=g)).bfloat16()
    keys = (torch.randn(batch, tokens, 576, generator=g) * 0.05).bfloat16()
    for first, last, factor in [(100, 110, 1.0), (200, 260, 4.0)]:
        keys[:, first:last] = (direction * factor).bfloat16()
    ql, qr = query[..., :512].contiguous(), query[..., 512:].contiguous()
    c, kr = keys[..., :512].contiguous(), keys[..., 512:].contiguous()
    scale = 1.0
    announce("mla_forward raised reference")
    out, lse = ops.mla_forward(ql.to(cuda), qr.to(cuda), c.to(cuda), kr.to(cuda), scale)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.mla_forward_unrounded(ql, qr, c, kr, scale, oracle.causal_mask(tokens))
    assert expected_lse.max() > 500 and expected_lse[..., :100].max() < 200
    torch.testing.assert_close(out.cpu().float(), expected, atol=8e-3, rtol=8e-3)
    worst = ((lse.cpu() - expected_lse).abs() / expected_lse.abs().clamp_min(1)).max().item()
    assert worst <= 1e-5


def test_absorbed_forward_closed_form_constant_fill(cuda):
    """benchmarks/attention/benchmark_mla.cu:38-47: O == 0.25, LSE[t] = 0.6614583 + ln(t+1)."""
    batch, tokens, heads = 1, 128, 8
    ql = torch.full((batch, tokens, heads, 512), 0.125).bfloat16()
    qr = torch.full((batch, tokens, heads, 64), -0.0625).bfloat16()
    c = torch.full((batch, tokens, 512), 0.25).bfloat16()
    kr = torch.full((batch, tokens, 64), 0.03125).bfloat16()
    out, lse = ops.mla_forward(ql.to(cuda), qr.to(cuda), c.to(cuda), kr.to(cuda), 1.0 / 24.0)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().float(), torch.full((batch, tokens, heads, 512), 0.25))
    expected = 0.6614583333 + torch.log(torch.arange(1, tokens + 1, dtype=torch.float32))
    assert (lse.cpu() - expected[None, None]).abs().max() <= 1e-4
