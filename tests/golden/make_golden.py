"""Writes the golden fixtures of this directory.

The reference holds no stored vectors for the attention path (its tests draw
inputs from the CUDA generator and compare against an in-process PyTorch
oracle), so these fixtures are produced by this repository's own CPU oracle,
``oracle/attention_oracle.py``, after the pins of ``tests/test_oracle_pins.py``
pass.  They freeze inputs (bf16 bit patterns) and fp32 expected outputs of one
small case per entry point, so that a later change of the oracle or of the
input generators cannot go unnoticed, and give the GPU tests data that does
not depend on any generator.

Run from the repository root:  python tests/golden/make_golden.py
"""

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from dscuda_amd.harness import configs  # noqa: E402
from oracle import attention_oracle as oracle  # noqa: E402

HERE = Path(__file__).resolve().parent


def bits(tensor):
    return tensor.contiguous().view(torch.int16).numpy().astype(np.uint16)


def main():
    # causal flash attention forward, GQA 4:2, D=64
    q, k, v, scale = configs.flash_forward_inputs(1, 64, 4, 2, 64, seed=101, factor=0.5)
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    np.savez_compressed(HERE / "flash_forward.npz", q=bits(q), k=bits(k), v=bits(v), scale=np.float32(scale),
                        out=out.numpy(), lse=lse.numpy())

    # per-head MLA prefill forward + backward, 128+64 | 128, ragged length
    q, k, v, scale = configs.mla_prefill_inputs(1, 45, 2, seed=102)
    dout = configs.mla_prefill_dout(1, 45, 2, 128, seed=103)
    out, lse = oracle.causal_attention_forward(q, k, v, scale)
    saved = out.bfloat16()
    dq, dk, dv = oracle.attention_backward(dout, saved, lse, q, k, v, scale)
    np.savez_compressed(HERE / "mla_prefill.npz", q=bits(q), k=bits(k), v=bits(v), dout=bits(dout),
                        saved_out=bits(saved), scale=np.float32(scale), out=out.numpy(), lse=lse.numpy(),
                        dq=dq.numpy(), dk=dk.numpy(), dv=dv.numpy())

    # absorbed forward + backward, reference test shape (2, 17, 3)
    ql, qr, c, kr, scale = configs.mla_absorbed_inputs(2, 17, 3, seed=104)
    g = torch.Generator().manual_seed(105)
    dout = (torch.randn(2, 17, 3, 512, generator=g) * 0.2).bfloat16()
    mask = oracle.causal_mask(17)
    out, lse = oracle.mla_forward_unrounded(ql, qr, c, kr, scale, mask)
    saved = out.bfloat16()
    grads = oracle.mla_backward_unrounded(dout, saved, lse, ql, qr, c, kr, scale, mask)
    np.savez_compressed(HERE / "mla_absorbed.npz", ql=bits(ql), qr=bits(qr), c=bits(c), kr=bits(kr), dout=bits(dout),
                        saved_out=bits(saved), scale=np.float32(scale), out=out.numpy(), lse=lse.numpy(),
                        dql=grads[0].numpy(), dqr=grads[1].numpy(), dc=grads[2].numpy(), dkr=grads[3].numpy())

    # decode: lengths 1 and 70 (a page boundary + 6), 4 heads
    g = torch.Generator().manual_seed(106)
    query = (torch.randn(2, 1, 4, 576, generator=g) * 0.5).bfloat16()
    cache = (torch.randn(2, 70, 576, generator=g) * 0.5).bfloat16()
    lengths = torch.tensor([1, 70], dtype=torch.int32)
    scale = configs.c_float(192 ** -0.5)
    out, lse = oracle.mla_decode_unrounded(query, cache, lengths, scale)
    np.savez_compressed(HERE / "mla_decode.npz", query=bits(query), cache=bits(cache), lengths=lengths.numpy(),
                        scale=np.float32(scale), out=out.numpy(), lse=lse.numpy())
    for path in sorted(HERE.glob("*.npz")):
        print(path.name, path.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
