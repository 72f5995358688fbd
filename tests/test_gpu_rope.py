"""The rotary-embedding kernel (dscuda_rope_apply) against the oracle's statement of the convention (complex
multiplication in fp64, pinned by closed forms in tests/test_oracle_pins.py), rounded to bf16.  The kernel computes
in fp32 (fp32 sine / cosine of an fp64-exact angle, unfused products), so its result differs from the correctly
rounded one only where fp32 rounding moves a value across a bf16 rounding boundary: a small fraction of the
elements, each off by one bf16 step, or by less than 1e-5 where the two products of a rotation cancel."""

import pytest
import torch

from dscuda_amd.harness import ops
from oracle import attention_oracle as oracle
from tests.parity import announce

pytestmark = pytest.mark.gpu


def _expected(x, offset, size, theta=10000.0, start=None):
    out = x.double().clone()
    for b in range(x.shape[0]):
        first = 0 if start is None else int(start[b])
        out[b:b + 1, :, :, offset:offset + size] = oracle.apply_rope(x[b:b + 1, :, :, offset:offset + size], theta, first)
    return out.float().bfloat16()


def _compare(got, expected):
    got, expected = got.cpu(), expected
    different = (got.view(torch.int16) != expected.view(torch.int16))
    fraction = different.float().mean().item()
    assert fraction <= 3e-4, f"{fraction:.2e} of the elements differ"
    if different.any():
        # ... and then by one bf16 step, or by next to nothing in absolute terms where the two products cancel
        a, b = got[different].float(), expected[different].float()
        assert ((a - b).abs() <= torch.maximum(b.abs() * 2.0 ** -7, torch.tensor(1e-5))).all()


@pytest.mark.parametrize("shape,offset,size", [
    ((1, 4096, 4, 192), 128, 64),      # the rope columns of per-head Q / K (workloads 2 and 3), 4 of the heads
    ((2, 257, 3, 64), 0, 64),          # q_rope of the absorbed form, ragged
    ((3, 33, 1, 64), 0, 64),           # k_rope: one shared head
    ((1, 16384, 1, 192), 128, 64),     # positions of workload 5
    ((2, 50, 5, 40), 8, 32),           # another width: 16 pairs, four groups of lanes
    ((1, 7, 2, 8), 2, 4),
])
def test_rope_matches_the_oracle(cuda, shape, offset, size):
    announce("rope", dict(shape=shape, offset=offset, size=size))
    g = torch.Generator().manual_seed(77)
    x = (torch.randn(shape, generator=g) * 0.5).bfloat16()
    got = ops.rope_apply(x.to(cuda), offset, size)
    torch.cuda.synchronize()
    expected = _expected(x, offset, size)
    _compare(got, expected)
    # columns outside the slice are untouched
    untouched = torch.ones(shape[-1], dtype=torch.bool)
    untouched[offset:offset + size] = False
    assert torch.equal(got.cpu()[..., untouched], x[..., untouched])


def test_rope_with_start_positions(cuda):
    """The one new token of a decode step sits at position length - 1 of its sequence."""
    announce("rope with start positions")
    g = torch.Generator().manual_seed(78)
    x = (torch.randn(4, 1, 16, 64, generator=g) * 0.5).bfloat16()
    start = torch.tensor([0, 1023, 5000, 8191], dtype=torch.int32)
    got = ops.rope_apply(x.to(cuda), 0, 64, positions=start.to(cuda))
    torch.cuda.synchronize()
    _compare(got, _expected(x, 0, 64, start=start))


def test_rope_is_a_rotation(cuda):
    """Pair norms are preserved, and rotating by theta then reading position 0 changes nothing."""
    g = torch.Generator().manual_seed(79)
    x = (torch.randn(1, 512, 2, 64, generator=g) * 0.5).bfloat16()
    got = ops.rope_apply(x.to(cuda).clone(), 0, 64).cpu().float()
    before = x.float().reshape(1, 512, 2, 32, 2).pow(2).sum(-1)
    after = got.reshape(1, 512, 2, 32, 2).pow(2).sum(-1)
    torch.testing.assert_close(after, before, atol=2e-2, rtol=2e-2)
    assert torch.equal(got[:, 0], x.float()[:, 0])


def test_rope_rejects_bad_slices(cuda):
    x = torch.zeros(1, 4, 2, 64, device=cuda, dtype=torch.bfloat16)
    for offset, size in ((0, 48), (1, 32), (48, 32), (0, 0)):
        with pytest.raises(RuntimeError):
            ops.rope_apply(x, offset, size)
