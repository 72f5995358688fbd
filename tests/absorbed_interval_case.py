"""One absorbed backward case in a process of its own, run by test_gpu_backward.py with DSCUDA_AMD_KEY_INTERVAL_TILES
set: the variable is read once per process, and without it the interval cut of the key gradients only starts at
sizes no test could check against the oracle.

usage: python -m tests.absorbed_interval_case BATCH TOKENS HEADS"""

import os
import sys

import torch

from dscuda_amd.harness import common, configs, ops
from oracle import attention_oracle as oracle
from tests.parity import assert_close_bf16


def main(batch, tokens, heads):
    assert int(os.environ["DSCUDA_AMD_KEY_INTERVAL_TILES"]) > 0
    cuda = torch.device("cuda:0")
    ql, qr, c, kr, scale = configs.mla_absorbed_inputs(batch, tokens, heads)
    g = torch.Generator().manual_seed(78)
    dout = (torch.randn(batch, tokens, heads, 512, generator=g) * (0.2 if heads <= 32 else 0.05)).bfloat16()
    mask = oracle.causal_mask(tokens)
    out, lse = oracle.mla_forward(ql, qr, c, kr, scale, mask)
    grads = ops.mla_backward(dout.to(cuda), out.to(cuda), lse.to(cuda), ql.to(cuda), qr.to(cuda), c.to(cuda),
                             kr.to(cuda), scale)
    torch.cuda.synchronize()
    expected = oracle.mla_backward_unrounded(dout, out, lse, ql, qr, c, kr, scale, mask)
    for name, actual, reference in zip(("dq_latent", "dq_rope", "dlatent", "dk_rope"), grads, expected):
        assert_close_bf16(name, actual.cpu(), reference)
    print("interval cut ok", batch, tokens, heads, flush=True)


if __name__ == "__main__":
    main(*map(int, sys.argv[1:4]))
    common.leave()
