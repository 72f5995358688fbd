"""One entry point for runtime comparison tables, after the reference's
``benchmarks/run.py``: every operation of a family is checked against a PyTorch
expression of the same mathematics on the same GPU, then both are timed by HIP
graph replay and reported in the six-column table (``report.py``).

    python -m dscuda_amd.harness.run mla --suite quick
    python -m dscuda_amd.harness.run all --suite full --output /tmp/runtime
    python -m dscuda_amd.harness.run mla_prefill --suite metric --operation forward --no-reference

Families: ``flash_attention`` and ``mla`` (the reference's shapes,
``benchmarks/flash_attention.py:44-57``, ``benchmarks/mla.py:38-49``) and
``mla_prefill`` (the per-head 192/192/128 form of the headline metric, which
the reference does not have).  Suites: ``quick``, ``full`` (the reference's),
``metric`` (the workloads of the headline metric; PyTorch in fp32 needs tens of
GB there, so ``--no-reference`` is usual).  The PyTorch side is
``torch.nn.functional.scaled_dot_product_attention`` in fp32 and autograd
through it: a library routine, not this repository's test oracle.  Parity
against the oracle is the business of ``tests/``; the check here only guards
the timing against a broken kernel, with the reference harness's tolerances
(``benchmarks/mla.py:100,124``, ``benchmarks/flash_attention.py:112-113``).
"""

from __future__ import annotations

import argparse
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parents[2]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

from dscuda_amd.harness import configs, report  # noqa: E402

FAMILIES = ("flash_attention", "mla", "mla_prefill")


def _close(actual, expected, atol, rtol):
    import torch
    actual = (actual,) if isinstance(actual, torch.Tensor) else tuple(actual)
    assert len(actual) == len(expected)
    for index, (got, want) in enumerate(zip(actual, expected)):
        a = atol[index] if isinstance(atol, tuple) else atol
        r = rtol[index] if isinstance(rtol, tuple) else rtol
        torch.testing.assert_close(got.float(), want.float(), atol=a, rtol=r)


def _sdpa(query, key, value, scale, mask=None, causal=False):
    """fp32 attention on [B,T,H,D] tensors (heads broadcast if key has one) -> (O [B,T,H,Dv], LSE [B,H,T])."""
    import torch
    q, k, v = (x.float().transpose(1, 2) for x in (query, key, value))
    if k.shape[1] != q.shape[1]:
        k = k.repeat_interleave(q.shape[1] // k.shape[1], dim=1)
        v = v.repeat_interleave(q.shape[1] // v.shape[1], dim=1)
    out = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, is_causal=causal, scale=scale)
    scores = q @ k.transpose(-1, -2) * scale
    if causal:
        keep = torch.ones(q.shape[-2], k.shape[-2], device=q.device, dtype=torch.bool).tril()
        scores = scores.masked_fill(~keep, -torch.inf)
    elif mask is not None:
        scores = scores.masked_fill(~mask, -torch.inf)
    return out.transpose(1, 2), scores.logsumexp(-1)


def flash_cases(args):
    import torch
    from dscuda_amd.harness import ops
    if args.suite == "quick":
        shapes = [(1, 512, 8, kv, 128) for kv in (8, 2, 1)]
    elif args.suite == "metric":
        shapes = [(1, 512, 8, 8, 64)]
    else:
        shapes = [(b, t, 8, kv, 128) for b in (1, 4) for t in (128, 256, 512, 1024, 2048) for kv in (8, 2, 1)]
    for b, t, hq, hkv, d in shapes:
        q, k, v, scale = configs.flash_forward_inputs(b, t, hq, hkv, d, seed=0, factor=0.5)
        q, k, v = q.cuda(), k.cuda(), v.cuda()
        out, lse = torch.empty_like(q), torch.empty(b, hq, t, device="cuda")
        functions = {"custom": lambda q=q, k=k, v=v, out=out, lse=lse, scale=scale: ops.flash_forward(q, k, v, scale, out, lse)}
        check = None
        if not args.no_reference:
            reference = lambda q=q, k=k, v=v, scale=scale: _sdpa(q, k, v, scale, causal=True)  # noqa: E731
            functions["PyTorch"] = reference
            expected = tuple(x.detach() for x in reference())
            check = lambda result, expected=expected: _close(result, expected, (1e-2, 1e-4), (1e-2, 1e-5))  # noqa: E731
        yield report.Operation(f"B={b},T={t},Hq={hq},Hkv={hkv},D={d}", "bf16", "forward", functions, check)


def mla_cases(args):
    import torch
    from dscuda_amd.harness import ops
    shapes = [("prefill", 1, 128, 8), ("decode", 2, 1024, 16)]
    if args.suite == "metric":
        shapes = [("decode", 64, 0, 128)]
    elif args.suite != "quick":
        shapes += [("prefill", 2, 257, 4), ("prefill", 1, 512, 8), ("decode", 1, 256, 16), ("decode", 4, 4096, 32)]
    for mode, b, t, h in shapes:
        if mode == "decode" and t == 0:   # the metric's decode workload: lengths ~ U[1024, 8192]
            data = configs.mla_decode_inputs()
            lengths = [int(x) for x in data["lengths"]]
            t = max(lengths)
            packed_query, paged, table = data["query"].cuda(), data["paged"].cuda(), data["table"].cuda()
            cache, scale = data["cache"].cuda(), data["scale"]
        else:
            q_lat, q_rope, latent, k_rope, scale = (x.cuda() if hasattr(x, "cuda") else x for x in
                                                     configs.mla_absorbed_inputs(b, t, h, query_tokens=None if mode == "prefill" else 1))
            lengths = configs.harness_decode_lengths(b, t, test=False)
            if mode == "decode":
                packed_query = torch.cat((q_lat, q_rope), -1).contiguous()
                cache = torch.cat((latent, k_rope), -1)
                paged, table = configs.pack_cache(cache, 64)
        size = f"B={b},Q={t if mode == 'prefill' else 1},KV={t},H={h},C=512,RoPE=64"
        if mode == "prefill":
            out = torch.empty(b, t, h, 512, device="cuda", dtype=torch.bfloat16)
            lse = torch.empty(b, h, t, device="cuda")
            inputs = (q_lat, q_rope, latent, k_rope)
            functions = {"custom": lambda i=inputs, s=scale, o=out, l=lse: ops.mla_forward(*i, s, o, l)}

            def pytorch_forward(i=inputs, s=scale):
                ql, qr, c, kr = i
                return _sdpa(torch.cat((ql, qr), -1), torch.cat((c, kr), -1)[:, :, None], c[:, :, None], s, causal=True)

            check, saved = None, None
            if not args.no_reference:
                functions["PyTorch"] = pytorch_forward
                saved = tuple(x.detach() for x in pytorch_forward())
                check = lambda result, e=saved: _close(result, e, (8e-3, 1e-4), (8e-3, 1e-4))  # noqa: E731
            yield report.Operation(size, "bf16", "forward", functions, check)

            generator = torch.Generator().manual_seed(2027)
            dout = (torch.randn(out.shape, generator=generator) * 0.2).bfloat16().cuda()
            ops.mla_forward(*inputs, scale, out, lse)
            torch.cuda.synchronize()
            saved_out, saved_lse = out.clone(), lse.clone()
            grads = tuple(torch.empty_like(x) for x in inputs)
            functions = {"custom": lambda: ops.mla_backward(dout, saved_out, saved_lse, *inputs, scale, grads)}
            check = None
            if not args.no_reference:
                def pytorch_backward(i=inputs, s=scale):
                    leaves = tuple(x.float().detach().requires_grad_() for x in i)
                    with torch.enable_grad():
                        ql, qr, c, kr = leaves
                        result, _ = _sdpa(torch.cat((ql, qr), -1), torch.cat((c, kr), -1)[:, :, None], c[:, :, None], s,
                                          causal=True)
                        return torch.autograd.grad(result, leaves, dout.float())
                functions["PyTorch"] = pytorch_backward
                expected = tuple(x.detach() for x in pytorch_backward())
                check = lambda result, e=expected: _close(result, e, 1e-2, 1e-2)  # noqa: E731
            yield report.Operation(size, "bf16", "backward", functions, check)
        else:
            length_tensor = torch.tensor(lengths, device="cuda", dtype=torch.int32)
            workspace = ops.mla_decode_workspace(b, h, 8, 512, "cuda")
            out = torch.empty(b, 1, h, 512, device="cuda", dtype=torch.bfloat16)
            lse = torch.empty(b, h, 1, device="cuda")
            functions = {"custom": lambda: ops.mla_decode(packed_query, paged, table, length_tensor, scale, splits=8,
                                                          workspace=workspace, out=out, lse=lse)}
            check = None
            if not args.no_reference:
                mask = (torch.arange(t, device="cuda")[None] < length_tensor[:, None])[:, None, None]

                def pytorch_decode():
                    return _sdpa(packed_query, cache[:, :, None], cache[:, :, None, :512], scale, mask=mask)
                functions["PyTorch"] = pytorch_decode
                expected = tuple(x.detach() for x in pytorch_decode())
                check = lambda result, e=expected: _close(result, e, (8e-3, 1e-4), (8e-3, 1e-4))  # noqa: E731
            shown = lengths if len(lengths) <= 8 else f"U[{min(lengths)},{max(lengths)}] sum {sum(lengths)}"
            yield report.Operation(size + f",lengths={shown},page=64,custom_splits=8", "bf16", "decode", functions, check)


def mla_prefill_cases(args):
    import torch
    from dscuda_amd.harness import ops
    shapes = {"quick": [(1, 1024, 16)], "full": [(1, 1024, 16), (1, 2048, 32), (2, 4096, 16)],
              "metric": [(1, 4096, 128)]}[args.suite]
    for b, s, h in shapes:
        q, k, v, scale = configs.mla_prefill_inputs(b, s, h, seed=1)
        q, k, v = q.cuda(), k.cuda(), v.cuda()
        out = torch.empty(b, s, h, 128, device="cuda", dtype=torch.bfloat16)
        lse = torch.empty(b, h, s, device="cuda")
        size = f"B={b},S={s},H={h},d_qk=192,d_v=128"
        functions = {"custom": lambda: ops.mla_prefill_forward(q, k, v, scale, out, lse)}
        check = None
        if not args.no_reference:
            reference = lambda: _sdpa(q, k, v, scale, causal=True)  # noqa: E731
            functions["PyTorch"] = reference
            expected = tuple(x.detach() for x in reference())
            check = lambda result, e=expected: _close(result, e, (1e-2, 1e-4), (1e-2, 1e-4))  # noqa: E731
        yield report.Operation(size, "bf16", "forward", functions, check,
                               notes={"flops": configs.forward_flops(b, h, s, 192, 128)})

        dout = configs.mla_prefill_dout(b, s, h, 128, seed=2).cuda()
        ops.mla_prefill_forward(q, k, v, scale, out, lse)
        torch.cuda.synchronize()
        saved_out, saved_lse = out.clone(), lse.clone()
        grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
        workspace = ops.mla_prefill_backward_workspace(b, s, h, 192, 128, "cuda")
        functions = {"custom": lambda: ops.mla_prefill_backward(dout, saved_out, saved_lse, q, k, v, scale, workspace, grads)}
        check = None
        if not args.no_reference:
            def pytorch_backward():
                leaves = tuple(x.float().detach().requires_grad_() for x in (q, k, v))
                with torch.enable_grad():
                    result, _ = _sdpa(*leaves, scale, causal=True)
                    return torch.autograd.grad(result, leaves, dout.float())
            functions["PyTorch"] = pytorch_backward
            expected = tuple(x.detach() for x in pytorch_backward())
            check = lambda result, e=expected: _close(result, e, 2e-2, 2e-2)  # noqa: E731
        yield report.Operation(size, "bf16", "backward", functions, check,
                               notes={"flops": configs.backward_flops(b, h, s, 192, 128)})


CASES = {"flash_attention": flash_cases, "mla": mla_cases, "mla_prefill": mla_prefill_cases}


class Graph:
    """`operations` back-to-back calls of one backend captured into a HIP graph
    (``benchmarks/common.py:64-72``); every entry point of the library may be
    captured: it allocates nothing and does not synchronise."""

    def __init__(self, function, operations):
        import torch
        for _ in range(3):
            function()
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=torch.cuda.current_stream()):
            for _ in range(operations):
                self.output = function()


def measure(operation, args):
    """Per-call microseconds of every backend, `args.trials` samples each (``benchmarks/common.py:75-111``)."""
    import torch
    with torch.no_grad():
        graphs = {name: Graph(call, args.graph_operations) for name, call in operation.functions.items()}
        for graph in graphs.values():
            graph.graph.replay()
            torch.cuda.synchronize()
            if operation.check:
                operation.check(graph.output)
        deadline = time.perf_counter() + args.warmup_ms / 1000
        while time.perf_counter() < deadline:
            for graph in graphs.values():
                graph.graph.replay()
            torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

        def elapsed(graph, repeats):
            start.record()
            for _ in range(repeats):
                graph.graph.replay()
            stop.record()
            stop.synchronize()
            return start.elapsed_time(stop)

        repeats = {name: report.repeats_for(args.sample_ms, elapsed(graph, 3) / 3) for name, graph in graphs.items()}
        samples = {name: [] for name in graphs}
        for trial in range(args.trials):
            for name in report.trial_order(graphs, trial):
                samples[name].append(1000 * elapsed(graphs[name], repeats[name]) / (repeats[name] * args.graph_operations))
        for graph in graphs.values():
            if operation.check:
                operation.check(graph.output)
    return samples


def main(argv=None):
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("family", choices=(*FAMILIES, "all"))
    parser.add_argument("--suite", choices=("quick", "full", "metric"), default="quick")
    parser.add_argument("--operation", help="run only this operation: forward, backward or decode")
    parser.add_argument("--no-reference", action="store_true", help="time the custom kernels only")
    parser.add_argument("--graph-operations", type=int, default=10)
    parser.add_argument("--warmup-ms", type=int, default=1000)
    parser.add_argument("--sample-ms", type=int, default=20)
    parser.add_argument("--trials", type=int, default=9)
    parser.add_argument("--output", default=str(ROOT / "build" / "runtime"), help="directory of the report files")
    args = parser.parse_args(argv)

    import torch
    if not torch.cuda.is_available():
        sys.exit("run.py needs a GPU")
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for family in (FAMILIES if args.family == "all" else (args.family,)):
            rows, samples = [], []
            for operation in CASES[family](args):
                if args.operation and operation.name != args.operation:
                    continue
                for backend, function in operation.functions.items():
                    try:
                        result = function()
                        stream.synchronize()   # surface asynchronous faults here, outside the timed replay
                        if operation.check:
                            operation.check(result)
                    except (AssertionError, RuntimeError) as error:
                        raise type(error)(f"{family}: {operation.size}, {operation.dtype}, {operation.name}, {backend}\n"
                                          f"{error}") from error
                timings = measure(operation, args)
                rows.extend(report.record(operation, timings))
                samples.append(dict(size=operation.size, dtype=operation.dtype, operation=operation.name,
                                    samples_us=timings, **operation.notes))
            stream.synchronize()
            if not rows:
                parser.error("No matching operations.")
            environment = {"gpu": torch.cuda.get_device_name(), "torch": torch.__version__, "hip": torch.version.hip}
            print(report.save_report(args.output, family, rows, samples, environment), end="")


if __name__ == "__main__":
    main()
