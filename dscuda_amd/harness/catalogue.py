"""What the runtime harness can run: a catalogue of workloads, and how each is bound to device buffers.

The catalogue is data.  ``select`` turns (family, suite, ``--test``, ``--operation``) into a list of ``Workload``
records without touching a GPU, so the choice of shapes is testable on any machine; ``bind`` then allocates the
buffers of one workload and returns a ``Bound`` object that knows how to call the library (backend ``custom``)
and, when asked, a PyTorch expression of the same mathematics (backend ``PyTorch``:
``torch.nn.functional.scaled_dot_product_attention`` in fp32 and autograd through it -- a library routine, not this
repository's test oracle), and how closely the two must agree.

Shapes, input scaling, label text and tolerances are those of the reference's harness, because its tables are what
this one's are compared with: ``benchmarks/mla.py:34-61,100-125`` (MLA forward / backward / decode, lengths
``max(1, t - i*t/(2b))``, 0.25 * N(0,1) inputs, 0.2 * N(0,1) output gradients, atol = rtol = 8e-3 for O and 1e-4 for
LSE, 1e-2 for gradients) and ``benchmarks/flash_attention.py:41-57,112-113`` (0.5 * N(0,1) inputs, O 1e-2 / 1e-2,
LSE 1e-4 / 1e-5).  Two additions have no counterpart there: the family ``mla_prefill`` (the per-head 192/192/128
form) and the suite ``metric`` (the workloads of this repository's headline figures).
"""

from __future__ import annotations

from dataclasses import dataclass, field

from . import configs

FAMILIES = ("flash_attention", "mla", "mla_prefill")
SUITES = ("quick", "full", "h100", "metric")


@dataclass(frozen=True)
class Workload:
    family: str
    operation: str          # forward | backward | decode
    shape: tuple            # flash: (B, T, Hq, Hkv, D); mla: (B, T, H); mla_prefill: (B, S, H)
    test: bool = False      # the reference's --test variant (decode lengths start at 1 and end at T)

    @property
    def label(self) -> str:
        """The text of the table's first column."""
        if self.family == "flash_attention":
            b, t, hq, hkv, d = self.shape
            return f"B={b},T={t},Hq={hq},Hkv={hkv},D={d}"
        b, t, h = self.shape
        if self.family == "mla_prefill":
            return f"B={b},S={t},H={h},d_qk=192,d_v=128"
        queries = 1 if self.operation == "decode" else t
        text = f"B={b},Q={queries},KV={t if t else 'U[1024,8192]'},H={h},C=512,RoPE=64"
        if self.operation == "decode" and t:
            lengths = tuple(configs.harness_decode_lengths(b, t, test=self.test))
            text += f",lengths={lengths},page=64,custom_splits=8"
        elif self.operation == "decode":
            text += ",lengths~seed 3,page=64,custom_splits=8"
        return text


# ---- the catalogue --------------------------------------------------------------------------------------------

_FLASH = {
    "test": configs.FLASH_TEST,
    "quick": [(1, 512, 8, kv, 128) for kv in (8, 2, 1)],
    "full": [(b, t, 8, kv, 128) for b in (1, 4) for t in (128, 256, 512, 1024, 2048) for kv in (8, 2, 1)],
    "metric": [(1, 512, 8, 8, 64)],
}
_FLASH["h100"] = _FLASH["full"]   # the reference's h100 suite differs from full only in the references it loads

_MLA_PREFILL_SHAPES = {
    "test": configs.MLA_TEST_PREFILL,
    "quick": configs.MLA_FULL_PREFILL[:1],
    "full": configs.MLA_FULL_PREFILL,
    "h100": [],
    "metric": [],
}
_MLA_DECODE_SHAPES = {
    "test": configs.MLA_TEST_DECODE,
    "quick": configs.MLA_FULL_DECODE[:1],
    "full": configs.MLA_FULL_DECODE,
    "h100": [(1, 1024, 64), (4, 4096, 64), (4, 4096, 128), (8, 8192, 128)],   # benchmarks/mla.py:40-42
    "metric": [(64, 0, 128)],                                                  # KV 0: lengths ~ U[1024, 8192], seed 3
}
_PER_HEAD = {
    "test": [(1, 65, 2), (2, 257, 3)],
    "quick": [(1, 1024, 16)],
    "full": [(1, 1024, 16), (1, 2048, 32), (2, 4096, 16)],
    "h100": [(1, 4096, 128)],
    "metric": [(1, 4096, 128)],
}


def select(family: str, suite: str = "quick", test: bool = False, operation: str | None = None) -> list[Workload]:
    """The workloads of one family, in table order.  ``test`` replaces the suite's shapes by the small ragged ones
    the reference checks correctness on."""
    if family not in FAMILIES:
        raise ValueError(f"unknown family {family!r}; choose from {FAMILIES}")
    if suite not in SUITES:
        raise ValueError(f"unknown suite {suite!r}; choose from {SUITES}")
    key = "test" if test else suite
    chosen: list[Workload] = []
    if family == "flash_attention":
        chosen = [Workload(family, "forward", shape, test) for shape in _FLASH[key]]
    elif family == "mla":
        for shape in _MLA_PREFILL_SHAPES[key]:
            chosen += [Workload(family, "forward", shape, test), Workload(family, "backward", shape, test)]
        chosen += [Workload(family, "decode", shape, test) for shape in _MLA_DECODE_SHAPES[key]]
    else:
        for shape in _PER_HEAD[key]:
            chosen += [Workload(family, "forward", shape, test), Workload(family, "backward", shape, test)]
    if operation:
        chosen = [w for w in chosen if w.operation == operation]
    return chosen


# ---- binding to the device ------------------------------------------------------------------------------------

@dataclass
class Bound:
    """One workload with its buffers in device memory.  ``backends`` maps a backend name to a zero-argument callable
    that runs it once on the current stream and returns its outputs (tensors that later calls overwrite)."""
    workload: Workload
    backends: dict
    expected: tuple | None = None        # what every backend's outputs are compared with
    tolerance: tuple = ()                # (atol, rtol) per output
    facts: dict = field(default_factory=dict)
    dtype: str = "bf16"

    def verify(self, backend: str, outputs) -> None:
        """AssertionError when `outputs` of `backend` differ from the expected tensors by more than the tolerance."""
        import torch
        if self.expected is None:
            return
        outputs = (outputs,) if isinstance(outputs, torch.Tensor) else tuple(outputs)
        if len(outputs) != len(self.expected):
            raise AssertionError(f"{backend} returned {len(outputs)} tensors, expected {len(self.expected)}")
        for index, (got, want) in enumerate(zip(outputs, self.expected)):
            atol, rtol = self.tolerance[min(index, len(self.tolerance) - 1)]
            torch.testing.assert_close(got.float(), want.float(), atol=atol, rtol=rtol,
                                       msg=lambda text, i=index: f"output {i} of {backend}: {text}")


def _attention(query, key, value, scale, mask=None, causal=False):
    """fp32 attention on [B,T,H,D] tensors (a single key head is shared by all query heads) ->
    (O [B,T,H,Dv], LSE [B,H,T])."""
    import torch
    q, k, v = (x.float().transpose(1, 2) for x in (query, key, value))
    if k.shape[1] != q.shape[1]:
        repeat = q.shape[1] // k.shape[1]
        k, v = k.repeat_interleave(repeat, dim=1), v.repeat_interleave(repeat, dim=1)
    out = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, is_causal=causal, scale=scale)
    scores = q @ k.transpose(-1, -2) * scale
    if causal:
        scores = scores.masked_fill(~torch.ones(scores.shape[-2:], device=q.device, dtype=torch.bool).tril(), -torch.inf)
    elif mask is not None:
        scores = scores.masked_fill(~mask, -torch.inf)
    return out.transpose(1, 2), scores.logsumexp(-1)


def _gradients(forward, leaves, dout):
    """Gradients of `forward(*leaves)[0]` (fp32 leaves made from the bf16 inputs) for the output gradient `dout`."""
    import torch
    with torch.enable_grad():
        fresh = tuple(x.float().detach().requires_grad_() for x in leaves)
        return torch.autograd.grad(forward(*fresh)[0], fresh, dout.float())


def bind(workload: Workload, with_reference: bool = True, device: str = "cuda") -> Bound:
    binder = {"flash_attention": _bind_flash, "mla": _bind_mla, "mla_prefill": _bind_per_head}[workload.family]
    return binder(workload, with_reference, device)


def _bind_flash(workload, with_reference, device):
    import torch
    from . import ops
    b, t, hq, hkv, d = workload.shape
    q, k, v, scale = configs.flash_forward_inputs(b, t, hq, hkv, d, seed=0, factor=0.5)
    q, k, v = q.to(device), k.to(device), v.to(device)
    out, lse = torch.empty_like(q), torch.empty(b, hq, t, device=device)
    bound = Bound(workload, {"custom": lambda: ops.flash_forward(q, k, v, scale, out, lse)},
                  tolerance=((1e-2, 1e-2), (1e-4, 1e-5)), facts={"flops": configs.forward_flops(b, hq, t, d, d)})
    if with_reference:
        bound.backends["PyTorch"] = lambda: _attention(q, k, v, scale, causal=True)
        bound.expected = tuple(x.detach() for x in bound.backends["PyTorch"]())
    return bound


def _bind_mla(workload, with_reference, device):
    import torch
    from . import ops
    b, t, h = workload.shape
    if workload.operation == "decode":
        if t == 0:
            data = configs.mla_decode_inputs()
            lengths = data["lengths"].to(device)
            query, paged, table = data["query"].to(device), data["paged"].to(device), data["table"].to(device)
            cache, scale = data["cache"].to(device), data["scale"]
            tokens = cache.shape[1]
            facts = {"bytes": configs.decode_bytes(int(lengths.sum()), b, h)}
        else:
            q_lat, q_rope, latent, k_rope, scale = configs.mla_absorbed_inputs(b, t, h, query_tokens=1)
            query = torch.cat((q_lat, q_rope), -1).contiguous().to(device)
            cache = torch.cat((latent, k_rope), -1).to(device)
            paged, table = configs.pack_cache(cache, 64)
            lengths = torch.tensor(configs.harness_decode_lengths(b, t, test=workload.test), device=device, dtype=torch.int32)
            tokens = t
            facts = {"bytes": configs.decode_bytes(int(lengths.sum()), b, h)}
        workspace = ops.mla_decode_workspace(b, h, 8, 512, device)
        out = torch.empty(b, 1, h, 512, device=device, dtype=torch.bfloat16)
        lse = torch.empty(b, h, 1, device=device)
        bound = Bound(workload, {"custom": lambda: ops.mla_decode(query, paged, table, lengths, scale, splits=8,
                                                                  workspace=workspace, out=out, lse=lse)},
                      tolerance=((8e-3, 8e-3), (1e-4, 1e-4)), facts=facts)
        if with_reference:
            mask = (torch.arange(tokens, device=device)[None] < lengths[:, None])[:, None, None]
            bound.backends["PyTorch"] = lambda: _attention(query, cache[:, :, None], cache[:, :, None, :512], scale, mask=mask)
            bound.expected = tuple(x.detach() for x in bound.backends["PyTorch"]())
        return bound

    inputs = configs.mla_absorbed_inputs(b, t, h)
    scale = inputs[-1]
    q_lat, q_rope, latent, k_rope = (x.to(device) for x in inputs[:4])

    def reference_forward(ql, qr, c, kr):
        return _attention(torch.cat((ql, qr), -1), torch.cat((c, kr), -1)[:, :, None], c[:, :, None], scale, causal=True)

    out = torch.empty(b, t, h, 512, device=device, dtype=torch.bfloat16)
    lse = torch.empty(b, h, t, device=device)
    leaves = (q_lat, q_rope, latent, k_rope)
    if workload.operation == "forward":
        bound = Bound(workload, {"custom": lambda: ops.mla_forward(*leaves, scale, out, lse)},
                      tolerance=((8e-3, 8e-3), (1e-4, 1e-4)))
        if with_reference:
            bound.backends["PyTorch"] = lambda: reference_forward(*leaves)
            bound.expected = tuple(x.detach() for x in bound.backends["PyTorch"]())
        return bound
    generator = torch.Generator().manual_seed(2027)
    dout = (torch.randn(out.shape, generator=generator) * 0.2).bfloat16().to(device)
    ops.mla_forward(*leaves, scale, out, lse)
    torch.cuda.synchronize()
    saved_out, saved_lse = out.clone(), lse.clone()
    grads = tuple(torch.empty_like(x) for x in leaves)
    bound = Bound(workload, {"custom": lambda: ops.mla_backward(dout, saved_out, saved_lse, *leaves, scale, grads)},
                  tolerance=((1e-2, 1e-2),))
    if with_reference:
        bound.backends["PyTorch"] = lambda: _gradients(reference_forward, leaves, dout)
        bound.expected = tuple(x.detach() for x in bound.backends["PyTorch"]())
    return bound


def _bind_per_head(workload, with_reference, device):
    import torch
    from . import ops
    b, s, h = workload.shape
    q, k, v, scale = configs.mla_prefill_inputs(b, s, h, seed=1)
    q, k, v = q.to(device), k.to(device), v.to(device)
    out = torch.empty(b, s, h, 128, device=device, dtype=torch.bfloat16)
    lse = torch.empty(b, h, s, device=device)

    def reference_forward(query, key, value):
        return _attention(query, key, value, scale, causal=True)

    if workload.operation == "forward":
        bound = Bound(workload, {"custom": lambda: ops.mla_prefill_forward(q, k, v, scale, out, lse)},
                      tolerance=((1e-2, 1e-2), (1e-4, 1e-4)), facts={"flops": configs.forward_flops(b, h, s, 192, 128)})
        if with_reference:
            bound.backends["PyTorch"] = lambda: reference_forward(q, k, v)
            bound.expected = tuple(x.detach() for x in bound.backends["PyTorch"]())
        return bound
    dout = configs.mla_prefill_dout(b, s, h, 128, seed=2).to(device)
    ops.mla_prefill_forward(q, k, v, scale, out, lse)
    torch.cuda.synchronize()
    saved_out, saved_lse = out.clone(), lse.clone()
    grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    workspace = ops.mla_prefill_backward_workspace(b, s, h, 192, 128, device)
    bound = Bound(workload, {"custom": lambda: ops.mla_prefill_backward(dout, saved_out, saved_lse, q, k, v, scale,
                                                                        workspace, grads)},
                  tolerance=((2e-2, 2e-2),), facts={"flops": configs.backward_flops(b, h, s, 192, 128)})
    if with_reference:
        bound.backends["PyTorch"] = lambda: _gradients(reference_forward, (q, k, v), dout)
        bound.expected = tuple(x.detach() for x in bound.backends["PyTorch"]())
    return bound
