"""The decode entry point that allocates nothing (dscuda_mla_decode_static) against the entry point that
takes a caller workspace (dscuda_mla_decode), through the C-ABI: two calls in a row on one GPU, the second
with a smaller input, so the second call finds the first call's partial results and plan in the built-in
workspace.  Integer/byte-exact bar: both entry points run the same kernels, so outputs must be equal bit
for bit; the first call is also checked against the fp32 oracle."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16, assert_close_lse

pytestmark = pytest.mark.gpu

STATIC_BYTES = 64 << 20


def _inputs(batch, tokens, heads, seed):
    g = torch.Generator().manual_seed(seed)
    lengths = torch.randint(max(1, tokens // 3), tokens + 1, (batch,), generator=g, dtype=torch.int64).to(torch.int32)
    query = (torch.randn(batch, 1, heads, 576, generator=g) * 0.5).bfloat16()
    cache = (torch.randn(batch, tokens, 576, generator=g) * 0.5).bfloat16()
    paged, table = configs.pack_cache(cache, 64)
    return query, cache, paged, table, lengths


def test_static_workspace_decode_matches_the_workspace_entry_point(cuda):
    scale = configs.c_float(192 ** -0.5)
    first_oracle_done = False
    # a call that cuts sequences over many workgroups, then a smaller one that leaves most of the first
    # call's slots and plan untouched, then one that does not cut at all
    for batch, tokens, heads, splits, seed in [(12, 3000, 128, 8, 101), (3, 700, 128, 4, 102), (5, 300, 16, 1, 103)]:
        query, cache, paged, table, lengths = _inputs(batch, tokens, heads, seed)
        assert ops.mla_library().workspace(batch, heads, splits, 512) * 4 <= STATIC_BYTES
        announce("mla_decode_static", dict(B=batch, KV=tokens, H=heads, splits=splits))
        on_gpu = [x.to(cuda) for x in (query, paged, table, lengths)]
        out = torch.full((batch, 1, heads, 512), float("nan"), device=cuda, dtype=torch.bfloat16)
        lse = torch.full((batch, heads, 1), float("nan"), device=cuda, dtype=torch.float32)
        ops.mla_decode_static(*on_gpu, scale, splits, out, lse)
        torch.cuda.synchronize()
        expected_out, expected_lse = ops.mla_decode(*on_gpu, scale, splits=splits)
        torch.cuda.synchronize()
        assert torch.equal(out, expected_out) and torch.equal(lse, expected_lse)
        if not first_oracle_done:
            oracle_out, oracle_lse = oracle.mla_decode_unrounded(query, cache, lengths, scale)
            assert_close_bf16("O", out, oracle_out)
            assert_close_lse("LSE", lse, oracle_lse)
            first_oracle_done = True


def test_static_workspace_decode_rejects_sizes_beyond_its_capacity(cuda):
    batch, heads, splits = 64, 128, 8     # 64*128*8*514 floats = 135 MB
    assert ops.mla_library().workspace(batch, heads, splits, 512) * 4 > STATIC_BYTES
    query, cache, paged, table, lengths = _inputs(batch, 64, heads, 104)
    out = torch.empty(batch, 1, heads, 512, device=cuda, dtype=torch.bfloat16)
    lse = torch.empty(batch, heads, 1, device=cuda, dtype=torch.float32)
    with pytest.raises(RuntimeError, match="exceed the built-in workspace"):
        ops.mla_decode_static(query.to(cuda), paged.to(cuda), table.to(cuda), lengths.to(cuda),
                              configs.c_float(192 ** -0.5), splits, out, lse)
    # a split count that fits is accepted for the same shape
    ops.mla_decode_static(query.to(cuda), paged.to(cuda), table.to(cuda), lengths.to(cuda),
                          configs.c_float(192 ** -0.5), 3, out, lse)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()


def test_static_workspace_decode_allocates_nothing_and_replays_from_a_graph(cuda):
    """Device memory in use is the same before and after warm calls (the driver's own count, which sees allocations
    of any library in the process), and the call, captured into a graph after one eager call, replays bit-equal to
    the workspace entry point on fresh buffer contents, with eager work between the replays."""
    scale = configs.c_float(192 ** -0.5)
    batch, tokens, heads, splits = 6, 1500, 128, 8
    query, cache, paged, table, lengths = _inputs(batch, tokens, heads, 105)
    static = [x.to(cuda) for x in (query, paged, table, lengths)]
    out = torch.empty(batch, 1, heads, 512, device=cuda, dtype=torch.bfloat16)
    lse = torch.empty(batch, heads, 1, device=cuda, dtype=torch.float32)
    announce("mla_decode_static: no allocation", dict(B=batch, KV=tokens, H=heads, splits=splits))
    ops.mla_decode_static(*static, scale, splits, out, lse)      # first call on the device: symbol address, attributes
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before = torch.cuda.memory_reserved()
    for _ in range(3):
        ops.mla_decode_static(*static, scale, splits, out, lse)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before and torch.cuda.memory_reserved() == reserved_before

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.mla_decode_static(*static, scale, splits, out, lse)
    for seed in (106, 107):
        fresh = _inputs(batch, tokens, heads, seed)
        for target, source in zip(static, (fresh[0], fresh[2], fresh[3], fresh[4])):
            target.copy_(source)
        out.fill_(float("nan"))
        lse.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        replayed_out, replayed_lse = out.clone(), lse.clone()
        expected_out, expected_lse = ops.mla_decode(*static, scale, splits=splits)    # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(replayed_out, expected_out) and torch.equal(replayed_lse, expected_lse)
