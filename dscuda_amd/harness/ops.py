"""Operator-level callers of the C-ABI entry points.

Each function takes torch tensors that already live on the GPU, allocates the
outputs with torch (the caller owns every buffer, as in
``benchmarks/mla.py:56-57,69,111``) and calls one ``dscuda_*`` symbol on
torch's current stream.  Signatures of the ctypes bindings are the ones the
reference harness declares (``benchmarks/mla.py:27-32``,
``benchmarks/flash_attention.py:36-37``).
"""

from __future__ import annotations

import ctypes

import torch

from .common import F, I, P, bind, checked, library, pointers, stream


def _require_cuda(*tensors):
    for tensor in tensors:
        if not tensor.is_cuda:
            raise RuntimeError("dscuda_amd operators need GPU tensors; there is no CPU path")
        if not tensor.is_contiguous():
            raise RuntimeError("dscuda_amd operators need contiguous tensors")


class _Mla:
    def __init__(self):
        lib = library("mla")
        self.lib = lib
        self.forward = bind(lib, "dscuda_mla_forward", [P] * 6 + [I] * 5 + [F, P])
        self.backward = bind(lib, "dscuda_mla_backward", [P] * 11 + [I] * 5 + [F, P])
        self.decode = bind(lib, "dscuda_mla_decode", [P] * 7 + [I] * 7 + [F, P])
        self.decode_plan_elements = bind(lib, "dscuda_mla_decode_plan_elements", [I] * 4, ctypes.c_size_t)
        self.decode_plan = bind(lib, "dscuda_mla_decode_plan", [P] * 2 + [I] * 4 + [P])
        self.decode_planned = bind(lib, "dscuda_mla_decode_planned", [P] * 8 + [I] * 7 + [F, P])
        self.decode_static = bind(lib, "dscuda_mla_decode_static", [P] * 6 + [I] * 7 + [F, P])
        self.workspace = bind(lib, "dscuda_mla_workspace_elements", [I] * 4, ctypes.c_size_t)
        self.rope_apply = bind(lib, "dscuda_rope_apply", [P] * 2 + [I] * 6 + [F, P])
        L = ctypes.c_longlong
        self.absorb_query = bind(lib, "dscuda_mla_absorb_query", [P] * 3 + [L, I] + [L] * 5 + [P])
        self.unabsorb_output = bind(lib, "dscuda_mla_unabsorb_output", [P] * 3 + [L, I] + [L] * 5 + [P])
        self.prefill_forward = bind(lib, "dscuda_mla_prefill_forward", [P] * 5 + [I] * 5 + [F, P])
        self.prefill_backward = bind(lib, "dscuda_mla_prefill_backward", [P] * 10 + [I] * 5 + [F, P])
        self.prefill_workspace = bind(
            lib, "dscuda_mla_prefill_backward_workspace_elements", [I] * 5, ctypes.c_size_t)
        self.prefill_workspace_limit = bind(lib, "dscuda_mla_prefill_backward_set_workspace_limit", [ctypes.c_size_t], None)
        self.key_interval_tiles = bind(lib, "dscuda_mla_backward_set_key_interval_tiles", [I], None)


class _Flash:
    def __init__(self):
        lib = library("flash_attention")
        self.lib = lib
        self.forward = bind(lib, "dscuda_flash_forward", [P] * 5 + [I] * 5 + [F, P])
        self.backward = bind(lib, "dscuda_flash_backward", [P] * 10 + [I] * 5 + [F, P])
        self.backward_workspace = bind(lib, "dscuda_flash_backward_workspace_elements", [I] * 5, ctypes.c_size_t)
        self.backward_workspace_limit = bind(lib, "dscuda_flash_backward_set_workspace_limit", [ctypes.c_size_t], None)


_mla = None
_flash = None


def mla_library() -> _Mla:
    global _mla
    if _mla is None:
        _mla = _Mla()
    return _mla


def flash_library() -> _Flash:
    global _flash
    if _flash is None:
        _flash = _Flash()
    return _flash


def flash_forward(query, key, value, scale, out=None, lse=None):
    """query [B,T,Hq,D], key/value [B,T,Hkv,D] bf16 -> (O [B,T,Hq,D] bf16, LSE [B,Hq,T] fp32)."""
    _require_cuda(query, key, value)
    b, t, hq, d = query.shape
    hkv = key.shape[2]
    out = torch.empty_like(query) if out is None else out
    lse = torch.empty(b, hq, t, device=query.device, dtype=torch.float32) if lse is None else lse
    lib = flash_library()
    checked(lib.lib, "flash", lib.forward(*pointers((out, lse, query, key, value)), b, t, hq, hkv, d, scale, stream()))
    return out, lse


def mla_prefill_forward(query, key, value, scale, out=None, lse=None):
    """query/key [B,S,H,d_qk], value [B,S,H,d_v] bf16 -> (O [B,S,H,d_v] bf16, LSE [B,H,S] fp32)."""
    _require_cuda(query, key, value)
    b, s, h, dqk = query.shape
    dv = value.shape[-1]
    out = torch.empty(b, s, h, dv, device=query.device, dtype=torch.bfloat16) if out is None else out
    lse = torch.empty(b, h, s, device=query.device, dtype=torch.float32) if lse is None else lse
    lib = mla_library()
    checked(lib.lib, "mla", lib.prefill_forward(
        *pointers((out, lse, query, key, value)), b, s, h, dqk, dv, scale, stream()))
    return out, lse


def mla_prefill_backward_workspace_elements(batch, seq, heads, dqk, dv):
    """fp32 elements of the per-head backward's workspace (dscuda_mla_prefill_backward_workspace_elements)."""
    return mla_library().prefill_workspace(batch, seq, heads, dqk, dv)


def mla_prefill_backward_set_workspace_limit(limit_bytes: int) -> None:
    """Process-wide bound on the dS blocks of one chunk of (batch, head) pairs; 0 restores the built-in 3 GiB."""
    mla_library().prefill_workspace_limit(int(limit_bytes))


def mla_backward_set_key_interval_tiles(tiles: int) -> None:
    """Force the interval cut of the absorbed backward's key-gradient pass (0: the library's own choice)."""
    mla_library().key_interval_tiles(int(tiles))


def mla_prefill_backward_workspace(batch, seq, heads, dqk, dv, device="cuda"):
    """fp32 workspace of the per-head backward: row statistics plus the bf16 dS blocks that the dK/dV kernel hands
    to the dQ pass (about S^2 bytes per (batch, head) pair, for as many pairs as one pass covers)."""
    elements = mla_prefill_backward_workspace_elements(batch, seq, heads, dqk, dv)
    return torch.empty(elements, device=device, dtype=torch.float32)


def mla_prefill_backward(dout, out, lse, query, key, value, scale, workspace=None, grads=None):
    """-> (dQ, dK [B,S,H,d_qk], dV [B,S,H,d_v]) bf16, overwritten."""
    _require_cuda(dout, out, lse, query, key, value)
    b, s, h, dqk = query.shape
    dv = value.shape[-1]
    lib = mla_library()
    if workspace is None:
        workspace = mla_prefill_backward_workspace(b, s, h, dqk, dv, query.device)
    if grads is None:
        grads = (torch.empty_like(query), torch.empty_like(key), torch.empty_like(value))
    checked(lib.lib, "mla", lib.prefill_backward(
        *pointers((*grads, dout, out, lse, query, key, value, workspace)), b, s, h, dqk, dv, scale, stream()))
    return grads


def mla_forward(query_latent, query_rope, kv_latent, key_rope, scale, out=None, lse=None):
    """Absorbed causal MLA forward (dscuda_mla_forward)."""
    _require_cuda(query_latent, query_rope, kv_latent, key_rope)
    b, t, h, c = query_latent.shape
    r = query_rope.shape[-1]
    out = torch.empty_like(query_latent) if out is None else out
    lse = torch.empty(b, h, t, device=query_latent.device, dtype=torch.float32) if lse is None else lse
    lib = mla_library()
    checked(lib.lib, "mla", lib.forward(
        *pointers((out, lse, query_latent, query_rope, kv_latent, key_rope)), b, t, h, c, r, scale, stream()))
    return out, lse


def mla_backward(dout, out, lse, query_latent, query_rope, kv_latent, key_rope, scale, grads=None):
    """Absorbed MLA backward (dscuda_mla_backward) -> (dq_lat, dq_rope, dlatent, dk_rope)."""
    _require_cuda(dout, out, lse, query_latent, query_rope, kv_latent, key_rope)
    b, t, h, c = query_latent.shape
    r = query_rope.shape[-1]
    if grads is None:
        grads = tuple(torch.empty_like(x) for x in (query_latent, query_rope, kv_latent, key_rope))
    lib = mla_library()
    checked(lib.lib, "mla", lib.backward(
        *pointers((*grads, dout, out, lse, query_latent, query_rope, kv_latent, key_rope)),
        b, t, h, c, r, scale, stream()))
    return grads


def mla_decode_workspace(batch, heads, splits, rank=512, device="cuda"):
    lib = mla_library()
    return torch.empty(lib.workspace(batch, heads, splits, rank), device=device, dtype=torch.float32)


def mla_decode(packed_query, paged_cache, block_table, lengths, scale, splits=8, rank=512,
               workspace=None, out=None, lse=None):
    """packed_query [B,1,H,C+R], paged_cache [blocks,page,1,C+R], block_table int32 [B,pages],
    lengths int32 [B] -> (O [B,1,H,C] bf16, LSE [B,H,1] fp32)."""
    _require_cuda(packed_query, paged_cache, block_table, lengths)
    b, _, h, width = packed_query.shape
    rope = width - rank
    page_size = paged_cache.shape[1]
    pages = block_table.shape[1]
    device = packed_query.device
    if workspace is None:
        workspace = mla_decode_workspace(b, h, splits, rank, device)
    out = torch.empty(b, 1, h, rank, device=device, dtype=torch.bfloat16) if out is None else out
    lse = torch.empty(b, h, 1, device=device, dtype=torch.float32) if lse is None else lse
    lib = mla_library()
    checked(lib.lib, "mla", lib.decode(
        *pointers((out, lse, packed_query, paged_cache, block_table, lengths, workspace)),
        b, h, rank, rope, page_size, pages, splits, scale, stream()))
    return out, lse


def mla_decode_static(packed_query, paged_cache, block_table, lengths, scale, splits, out, lse, rank=512):
    """dscuda_mla_decode_static: the decode call for callers that cannot allocate.  The caller passes every
    input and output; partial results go to the workspace built into the library."""
    _require_cuda(packed_query, paged_cache, block_table, lengths, out, lse)
    b, _, h, width = packed_query.shape
    lib = mla_library()
    checked(lib.lib, "mla", lib.decode_static(
        *pointers((out, lse, packed_query, paged_cache, block_table, lengths)),
        b, h, rank, width - rank, paged_cache.shape[1], block_table.shape[1], splits, scale, stream()))
    return out, lse


def mla_decode_plan(lengths, heads, splits=8, rank=512):
    """dscuda_mla_decode_plan: the int table a batch of cache lengths needs, built once on the device for any
    number of mla_decode_planned calls over the same lengths, head count and splits."""
    _require_cuda(lengths)
    lib = mla_library()
    batch = lengths.numel()
    plan = torch.empty(lib.decode_plan_elements(batch, heads, splits, rank), device=lengths.device, dtype=torch.int32)
    checked(lib.lib, "mla", lib.decode_plan(plan.data_ptr(), lengths.data_ptr(), batch, heads, rank, splits, stream()))
    return plan


def mla_decode_planned(packed_query, paged_cache, block_table, lengths, plan, scale, splits=8, rank=512,
                       workspace=None, out=None, lse=None):
    """dscuda_mla_decode_planned: mla_decode with the plan of mla_decode_plan."""
    _require_cuda(packed_query, paged_cache, block_table, lengths, plan)
    b, _, h, width = packed_query.shape
    device = packed_query.device
    if workspace is None:
        workspace = mla_decode_workspace(b, h, splits, rank, device)
    out = torch.empty(b, 1, h, rank, device=device, dtype=torch.bfloat16) if out is None else out
    lse = torch.empty(b, h, 1, device=device, dtype=torch.float32) if lse is None else lse
    lib = mla_library()
    checked(lib.lib, "mla", lib.decode_planned(
        *pointers((out, lse, packed_query, paged_cache, block_table, lengths, workspace, plan)),
        b, h, rank, width - rank, paged_cache.shape[1], block_table.shape[1], splits, scale, stream()))
    return out, lse


def rope_apply(tensor, rope_offset=0, rope_size=None, theta=10000.0, positions=None):
    """Rotary position embedding in place on columns rope_offset .. rope_offset + rope_size - 1 of a contiguous
    [B,S,H,W] bf16 tensor (dscuda_rope_apply); positions: int32 [B] start positions or None.  Returns the tensor."""
    _require_cuda(tensor)
    if tensor.dim() != 4 or not tensor.is_contiguous() or tensor.dtype != torch.bfloat16:
        raise ValueError("rope_apply: a contiguous bf16 [B,S,H,W] tensor is required")
    b, s, h, w = tensor.shape
    rope_size = w - rope_offset if rope_size is None else rope_size
    if positions is not None:
        _require_cuda(positions)
        if positions.dtype != torch.int32 or positions.numel() != b:
            raise ValueError("rope_apply: positions must be int32 [B]")
    lib = mla_library()
    checked(lib.lib, "mla", lib.rope_apply(tensor.data_ptr(), positions.data_ptr() if positions is not None else None,
                                           b, s, h, w, rope_offset, rope_size, theta, stream()))
    return tensor


def _head_rows(name, tensor, width):
    """(tokens, heads, token stride, head stride) of a bf16 [..., H, >= width] view whose leading dimensions are
    laid out one behind the other and whose last dimension is contiguous."""
    if not tensor.is_cuda:
        raise RuntimeError("dscuda_amd operators need GPU tensors; there is no CPU path")
    if tensor.dtype != torch.bfloat16 or tensor.dim() < 3 or tensor.shape[-1] != width or tensor.stride(-1) != 1:
        raise ValueError(f"{name}: a bf16 [..., H, {width}] tensor with a contiguous last dimension is required")
    heads, token_stride = tensor.shape[-2], tensor.stride(-3)
    tokens = 1
    for size, stride in zip(reversed(tensor.shape[:-2]), reversed(tensor.stride()[:-2])):
        if size != 1 and stride != token_stride * tokens:
            raise ValueError(f"{name}: the token dimensions must be laid out one behind the other")
        tokens *= size
    return tokens, heads, token_stride, tensor.stride(-2)


def mla_absorb_query(query_nope, w_uk, out=None):
    """q_latent[..., h, :] = q_nope[..., h, :] @ w_uk[h]  (dscuda_mla_absorb_query).  query_nope: [..., H, 128] (may be
    the nope columns of a wider tensor), w_uk: [H, 128, 512] (may be a slice of wkv_b), out: [..., H, 512] (may be
    the latent columns of the packed decode query)."""
    tokens, heads, x_token, x_head = _head_rows("mla_absorb_query", query_nope, 128)
    if out is None:
        out = torch.empty(*query_nope.shape[:-1], 512, device=query_nope.device, dtype=torch.bfloat16)
    out_tokens, out_heads, y_token, y_head = _head_rows("mla_absorb_query", out, 512)
    if (out_tokens, out_heads) != (tokens, heads) or tuple(w_uk.shape) != (heads, 128, 512) or w_uk.stride()[1:] != (512, 1):
        raise ValueError("mla_absorb_query: shapes do not fit")
    lib = mla_library()
    checked(lib.lib, "mla", lib.absorb_query(out.data_ptr(), query_nope.data_ptr(), w_uk.data_ptr(), tokens, heads,
                                             x_token, x_head, y_token, y_head, w_uk.stride(0), stream()))
    return out


def mla_unabsorb_output(output_latent, w_uv, out=None):
    """out[..., h, :] = output_latent[..., h, :] @ w_uv[h].T  (dscuda_mla_unabsorb_output).  output_latent:
    [..., H, 512], w_uv: [H, 128, 512] (may be a slice of wkv_b), out: [..., H, 128]."""
    tokens, heads, x_token, x_head = _head_rows("mla_unabsorb_output", output_latent, 512)
    if out is None:
        out = torch.empty(*output_latent.shape[:-1], 128, device=output_latent.device, dtype=torch.bfloat16)
    out_tokens, out_heads, y_token, y_head = _head_rows("mla_unabsorb_output", out, 128)
    if (out_tokens, out_heads) != (tokens, heads) or tuple(w_uv.shape) != (heads, 128, 512) or w_uv.stride()[1:] != (512, 1):
        raise ValueError("mla_unabsorb_output: shapes do not fit")
    lib = mla_library()
    checked(lib.lib, "mla", lib.unabsorb_output(out.data_ptr(), output_latent.data_ptr(), w_uv.data_ptr(), tokens, heads,
                                                x_token, x_head, y_token, y_head, w_uv.stride(0), stream()))
    return out


def flash_backward_workspace(batch, seq, q_heads, kv_heads, dim, device="cuda"):
    """fp32 workspace of the flash-attention backward (dscuda_flash_backward_workspace_elements)."""
    elements = flash_library().backward_workspace(batch, seq, q_heads, kv_heads, dim)
    return torch.empty(elements, device=device, dtype=torch.float32)


def flash_backward(dout, out, lse, query, key, value, scale, workspace=None, grads=None):
    """Causal (grouped-query) attention backward (dscuda_flash_backward) -> (dQ [B,T,Hq,D], dK, dV [B,T,Hkv,D])."""
    _require_cuda(dout, out, lse, query, key, value)
    b, t, hq, d = query.shape
    hkv = key.shape[2]
    lib = flash_library()
    if workspace is None:
        workspace = flash_backward_workspace(b, t, hq, hkv, d, query.device)
    if grads is None:
        grads = (torch.empty_like(query), torch.empty_like(key), torch.empty_like(value))
    checked(lib.lib, "flash", lib.backward(
        *pointers((*grads, dout, out, lse, query, key, value, workspace)), b, t, hq, hkv, d, scale, stream()))
    return grads
