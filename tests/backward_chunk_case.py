"""One backward case in a process of its own, run by test_gpu_backward.py with DSCUDA_AMD_DS_BUDGET_BYTES set: the
budget is read once per process, so the chunked launches (several passes over groups of (batch, head) pairs that
share one set of dS blocks) can only be forced at a small size from outside.

usage: python -m tests.backward_chunk_case BATCH SEQ HEADS EXPECTED_PAIRS_PER_LAUNCH"""

import os
import sys

import torch

from dscuda_amd.harness import common, configs, ops
from oracle import attention_oracle as oracle
from tests.parity import assert_close_bf16


def main(batch, seq, heads, expected_chunk):
    cuda = torch.device("cuda:0")
    budget = int(os.environ["DSCUDA_AMD_DS_BUDGET_BYTES"])
    key_blocks, tiles = (seq + 127) // 128, (seq + 63) // 64
    blocks = sum(tiles - 2 * kb for kb in range(key_blocks))
    statistics = batch * heads * tiles * 128
    elements = ops.mla_prefill_backward_workspace(batch, seq, heads, 192, 128, cuda).numel()
    assert elements == statistics + expected_chunk * blocks * 4096, (elements, statistics, expected_chunk, blocks)
    assert expected_chunk * blocks * 16384 <= budget or expected_chunk == 1
    q, k, v, scale = configs.mla_prefill_inputs(batch, seq, heads, seed=31)
    dout = configs.mla_prefill_dout(batch, seq, heads, 128, seed=32)
    out_f, lse = oracle.causal_attention_forward(q, k, v, scale)
    out = out_f.bfloat16()
    dq, dk, dv = ops.mla_prefill_backward(dout.to(cuda), out.to(cuda), lse.to(cuda), q.to(cuda), k.to(cuda), v.to(cuda),
                                          scale)
    torch.cuda.synchronize()
    eq, ek, ev = oracle.attention_backward(dout, out, lse, q, k, v, scale)
    assert_close_bf16("dQ", dq.cpu(), eq)
    assert_close_bf16("dK", dk.cpu(), ek)
    assert_close_bf16("dV", dv.cpu(), ev)
    print("chunked backward ok", batch, seq, heads, expected_chunk, flush=True)


if __name__ == "__main__":
    main(*map(int, sys.argv[1:5]))
    common.leave()
