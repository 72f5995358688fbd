"""Every compute entry point of the C-ABI captured into a HIP graph and replayed.

The reference times all of its operations from inside a captured graph
(``benchmarks/common.py:68-76``), so capturability is part of the boundary: no
allocation, no synchronisation, no host-side dependence on the buffers' contents.
Each case captures one call on static buffers, then replays the graph after the
*contents* of the input buffers were replaced (twice, with different data and
eager work between the replays) and checks every replay against the fp32 oracle
of the data that was in the buffers at that time, and bit for bit against an
eager call on the same data."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from oracle import attention_oracle as oracle
from tests.parity import announce, assert_close_bf16, assert_close_lse

pytestmark = pytest.mark.gpu


def _replay_twice(cuda, make_inputs, call, check):
    """make_inputs(seed) -> tuple of CPU tensors; call(inputs_on_gpu, outputs or None) -> outputs;
    check(cpu_inputs, outputs) compares against the oracle."""
    first = make_inputs(0)
    static = [x.to(cuda) for x in first]
    outputs = call(static, None)             # eager: also performs the one-time function attribute set-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(static, outputs)
    for seed in (1, 2):
        fresh = make_inputs(seed)
        for target, source in zip(static, fresh):
            target.copy_(source)
        for tensor in outputs:
            tensor.fill_(float("nan")) if tensor.is_floating_point() else tensor.zero_()
        graph.replay()
        torch.cuda.synchronize()
        replayed = [x.clone() for x in outputs]
        check(fresh, replayed)
        eager = call(static, [torch.empty_like(x) for x in outputs])
        torch.cuda.synchronize()
        for a, b in zip(replayed, eager):
            assert torch.equal(a, b), "graph replay and eager call differ"


def test_graph_flash_forward(cuda):
    announce("graph capture: flash forward")

    def make(seed):
        return configs.flash_forward_inputs(2, 256, 8, 2, 128, seed=40 + seed, factor=0.5)[:3]

    scale = configs.c_float(128 ** -0.5)

    def call(x, outputs):
        out, lse = outputs if outputs else (None, None)
        return list(ops.flash_forward(x[0], x[1], x[2], scale, out, lse))

    def check(cpu, got):
        expected, expected_lse = oracle.causal_attention_forward(*cpu, scale)
        assert_close_bf16("O", got[0], expected)
        assert_close_lse("LSE", got[1], expected_lse)

    _replay_twice(cuda, make, call, check)


def test_graph_mla_prefill_forward_and_backward(cuda):
    announce("graph capture: mla prefill forward + backward")
    batch, seq, heads = 1, 384, 4
    scale = configs.c_float(192 ** -0.5)

    def make(seed):
        q, k, v, _ = configs.mla_prefill_inputs(batch, seq, heads, seed=50 + seed)
        dout = configs.mla_prefill_dout(batch, seq, heads, 128, seed=60 + seed)
        return q, k, v, dout

    workspace = ops.mla_prefill_backward_workspace(batch, seq, heads, 192, 128, cuda)

    def call(x, outputs):
        q, k, v, dout = x
        if outputs:
            out, lse, dq, dk, dv = outputs
        else:
            out = lse = None
            dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        out, lse = ops.mla_prefill_forward(q, k, v, scale, out, lse)
        ops.mla_prefill_backward(dout, out, lse, q, k, v, scale, workspace, (dq, dk, dv))
        return [out, lse, dq, dk, dv]

    def check(cpu, got):
        q, k, v, dout = cpu
        expected, expected_lse = oracle.causal_attention_forward(q, k, v, scale)
        assert_close_bf16("O", got[0], expected)
        assert_close_lse("LSE", got[1], expected_lse)
        # the backward consumed the kernel's own saved tensors
        reference = oracle.attention_backward(dout, got[0].cpu(), got[1].cpu(), q, k, v, scale)
        for name, actual, wanted in zip(("dQ", "dK", "dV"), got[2:], reference):
            assert_close_bf16(name, actual, wanted)

    _replay_twice(cuda, make, call, check)


def test_graph_mla_absorbed_forward_and_backward(cuda):
    announce("graph capture: absorbed mla forward + backward")
    batch, tokens, heads = 2, 65, 4
    scale = configs.c_float(576 ** -0.5)
    mask = oracle.causal_mask(tokens)

    def make(seed):
        ql, qr, c, kr, _ = configs.mla_absorbed_inputs(batch, tokens, heads, seed=70 + seed)
        g = torch.Generator().manual_seed(80 + seed)
        dout = (torch.randn(batch, tokens, heads, 512, generator=g) * 0.2).bfloat16()
        return ql, qr, c, kr, dout

    def call(x, outputs):
        ql, qr, c, kr, dout = x
        if outputs:
            out, lse = outputs[:2]
            grads = tuple(outputs[2:])
        else:
            out = lse = None
            grads = tuple(torch.empty_like(t) for t in (ql, qr, c, kr))
        out, lse = ops.mla_forward(ql, qr, c, kr, scale, out, lse)
        ops.mla_backward(dout, out, lse, ql, qr, c, kr, scale, grads)
        return [out, lse, *grads]

    def check(cpu, got):
        ql, qr, c, kr, dout = cpu
        expected, expected_lse = oracle.mla_forward_unrounded(ql, qr, c, kr, scale, mask)
        assert_close_bf16("O", got[0], expected)
        assert_close_lse("LSE", got[1], expected_lse)
        reference = oracle.mla_backward_unrounded(dout, got[0].cpu(), got[1].cpu(), ql, qr, c, kr, scale, mask)
        for name, actual, wanted in zip(("dq_latent", "dq_rope", "dlatent", "dk_rope"), got[2:], reference):
            assert_close_bf16(name, actual, wanted)

    _replay_twice(cuda, make, call, check)


@pytest.mark.parametrize("splits", [1, 8])
def test_graph_mla_decode(cuda, splits):
    """The decode call is several kernels with a device-side hand-over between them; the lengths change
    between the replays too, so the cut of the tile list is recomputed on the device each time."""
    announce("graph capture: mla decode", dict(splits=splits))
    batch, tokens, heads = 6, 1500, 128
    scale = configs.c_float(192 ** -0.5)
    table = torch.arange(batch * ((tokens + 63) // 64), dtype=torch.int32).reshape(batch, -1).to(cuda)
    workspace = ops.mla_decode_workspace(batch, heads, splits, 512, cuda)
    caches = {}

    def make(seed):
        g = torch.Generator().manual_seed(90 + seed)
        lengths = torch.randint(1, tokens + 1, (batch,), generator=g, dtype=torch.int64).to(torch.int32)
        query = (torch.randn(batch, 1, heads, 576, generator=g) * 0.5).bfloat16()
        cache = (torch.randn(batch, tokens, 576, generator=g) * 0.5).bfloat16()
        paged, _ = configs.pack_cache(cache, 64)
        caches[seed] = cache
        return query, paged, lengths, torch.tensor([seed])

    def call(x, outputs):
        query, paged, lengths, _ = x
        out, lse = outputs if outputs else (None, None)
        return list(ops.mla_decode(query, paged, table, lengths, scale, splits=splits, workspace=workspace,
                                   out=out, lse=lse))

    def check(cpu, got):
        query, _, lengths, seed = cpu
        expected, expected_lse = oracle.mla_decode_unrounded(query, caches[int(seed)], lengths, scale)
        assert_close_bf16("O", got[0], expected)
        assert_close_lse("LSE", got[1], expected_lse)

    _replay_twice(cuda, make, call, check)
