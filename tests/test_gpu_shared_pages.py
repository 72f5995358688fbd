"""Decode with a block table in which sequences share physical pages (a common prompt prefix stored once):
the layout a paged server produces.  The construction of the shared layout is checked on the CPU (gathering
the pages through the table must give back every sequence's logical cache); the GPU test then runs the decode
through the C-ABI on that table and compares with the fp32 oracle on the logical caches."""

import pytest
import torch

from dscuda_amd.harness import configs
from oracle import attention_oracle as oracle

PAGE = 64


def shared_prefix_layout(prefix_pages, tail_tokens, lone_tokens, seed=11, factor=0.25):
    """Sequences 0 .. len(tail_tokens)-1 share `prefix_pages` full pages and continue with their own tails;
    one more sequence of `lone_tokens` shares nothing.  Returns (logical [B, T, 576] zero padded, lengths,
    pool [blocks, PAGE, 1, 576], table int32 [B, pages])."""
    g = torch.Generator().manual_seed(seed)
    draw = lambda tokens: (torch.randn(tokens, 576, generator=g) * factor).bfloat16()   # noqa: E731
    prefix = draw(prefix_pages * PAGE)
    tails = [draw(tokens) for tokens in tail_tokens]
    lone = draw(lone_tokens)
    sequences = [torch.cat((prefix, tail)) for tail in tails] + [lone]
    lengths = [int(s.shape[0]) for s in sequences]
    longest = max(lengths)
    logical = torch.zeros(len(sequences), longest, 576, dtype=torch.bfloat16)
    for index, sequence in enumerate(sequences):
        logical[index, :sequence.shape[0]] = sequence

    def pages_of(tokens):
        count = (tokens.shape[0] + PAGE - 1) // PAGE
        padded = torch.zeros(count * PAGE, 576, dtype=torch.bfloat16)
        padded[:tokens.shape[0]] = tokens
        return list(padded.reshape(count, PAGE, 1, 576))

    pool, rows = pages_of(prefix), []
    for tail in tails:
        own = pages_of(tail)
        rows.append(list(range(prefix_pages)) + list(range(len(pool), len(pool) + len(own))))
        pool += own
    own = pages_of(lone)
    rows.append(list(range(len(pool), len(pool) + len(own))))
    pool += own
    width = max(len(row) for row in rows)
    table = torch.tensor([row + [0] * (width - len(row)) for row in rows], dtype=torch.int32)   # unused entries: any valid page
    return logical, lengths, torch.stack(pool).contiguous(), table


def test_shared_layout_reproduces_the_logical_caches():
    logical, lengths, pool, table = shared_prefix_layout(2, [172, 1, 64], 200)
    assert lengths == [300, 129, 192, 200]
    assert pool.shape[0] == 2 + 3 + 1 + 1 + 4 and table.shape == (4, 5)
    assert table[0, :2].tolist() == table[1, :2].tolist() == table[2, :2].tolist() == [0, 1]   # the prefix is stored once
    for index, length in enumerate(lengths):
        gathered = pool[table[index].long()].reshape(-1, 576)[:length]
        assert torch.equal(gathered, logical[index, :length])


@pytest.mark.gpu
@pytest.mark.parametrize("splits", [1, 8])
def test_decode_with_shared_prefix_pages(cuda, splits):
    from dscuda_amd.harness import ops
    from tests.parity import announce, assert_close_bf16, assert_close_lse
    logical, lengths, pool, table = shared_prefix_layout(2, [172, 1, 64], 200)
    heads = 32
    g = torch.Generator().manual_seed(12)
    query = (torch.randn(len(lengths), 1, heads, 576, generator=g) * 0.25).bfloat16()
    scale = configs.c_float(576 ** -0.5)
    lengths_t = torch.tensor(lengths, dtype=torch.int32)
    announce("mla_decode shared prefix", dict(B=len(lengths), H=heads, lengths=lengths, splits=splits, blocks=pool.shape[0]))
    out, lse = ops.mla_decode(query.to(cuda), pool.to(cuda), table.to(cuda), lengths_t.to(cuda), scale, splits=splits)
    torch.cuda.synchronize()
    expected, expected_lse = oracle.mla_decode_unrounded(query, logical, lengths_t, scale)
    assert_close_bf16("O", out, expected)
    assert_close_lse("LSE", lse, expected_lse)
