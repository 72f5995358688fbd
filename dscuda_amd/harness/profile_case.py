"""Runs one workload of the attention hot path a few times, for use under
``rocprofv3`` (kernel trace or one ``--pmc`` pass per run).  The counterpart of
the reference's standalone profiler mains (``benchmarks/attention/
benchmark_mla.cu``, ``benchmark_mla_decode.cu``, ``benchmark_flash_attention.cu``):
inputs are synthetic and generated on the GPU, one warm call precedes the
profiled ones.

    rocprofv3 --kernel-trace --stats -d out -- python3 dscuda_amd/harness/profile_case.py forward
    rocprofv3 --pmc SQ_BUSY_CU_CYCLES SQ_VALU_MFMA_BUSY_CYCLES -d out -- python3 dscuda_amd/harness/profile_case.py decode

Workloads: forward / backward (B=1, S, H=128, 192|128), decode (B=64, H=128,
lengths ~ U[1024, 8192] seed 3), flash (B=1, H=8, S=512, D=64), absorbed (the
reference's own prefill entry points, forward then backward, B=1, T=S, H heads,
512 latent + 64 rope), projection (the W_UK absorb and W_UV un-absorb of S tokens x
H heads), copy (a plain 16-byte-per-lane copy of 1 GiB, the calibration kernel for
FETCH_SIZE / WRITE_SIZE).  ``--data zero`` fills every input with zeros: the kernels
execute the same instructions, only the operands stop toggling, which separates what a
workload loses to the chip's power limit (the clock it is given) from what its schedule loses.
"""

from __future__ import annotations

import argparse
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[2]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def main():
    parser = argparse.ArgumentParser(description=__doc__)
    parser.add_argument("workload", choices=("forward", "backward", "decode", "flash", "absorbed", "projection", "copy"))
    parser.add_argument("--steps", type=int, default=3)
    parser.add_argument("--seq", type=int, default=4096)
    parser.add_argument("--heads", type=int, default=128)
    parser.add_argument("--data", choices=("random", "zero"), default="random")
    args = parser.parse_args()

    import torch

    from dscuda_amd.harness import configs, ops

    device = torch.device("cuda:0")
    generator = torch.Generator(device=device).manual_seed(1)

    def randn(shape, factor):
        if args.data == "zero":
            return torch.zeros(shape, device=device, dtype=torch.bfloat16)
        return (torch.randn(shape, device=device, generator=generator) * factor).bfloat16()

    if args.workload in ("forward", "backward"):
        s, h = args.seq, args.heads
        q, k, v = randn((1, s, h, 192), 0.5), randn((1, s, h, 192), 0.5), randn((1, s, h, 128), 0.5)
        scale = configs.c_float(192 ** -0.5)
        out = torch.empty(1, s, h, 128, device=device, dtype=torch.bfloat16)
        lse = torch.empty(1, h, s, device=device)
        ops.mla_prefill_forward(q, k, v, scale, out, lse)
        if args.workload == "forward":
            call = lambda: ops.mla_prefill_forward(q, k, v, scale, out, lse)
        else:
            dout = randn((1, s, h, 128), 1.0)
            grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
            workspace = ops.mla_prefill_backward_workspace(1, s, h, 192, 128, device)
            call = lambda: ops.mla_prefill_backward(dout, out, lse, q, k, v, scale, workspace, grads)
    elif args.workload == "decode":
        lengths, _ = configs.decode_lengths()
        b, h = lengths.numel(), args.heads
        pages = (int(lengths.max()) + 63) // 64
        query = randn((b, 1, h, 576), 0.5)
        paged = randn((b * pages, 64, 1, 576), 0.5)
        table = torch.arange(b * pages, device=device, dtype=torch.int32).reshape(b, pages)
        dl = lengths.to(device)
        workspace = ops.mla_decode_workspace(b, h, 8, 512, device)
        out = torch.empty(b, 1, h, 512, device=device, dtype=torch.bfloat16)
        lse = torch.empty(b, h, 1, device=device)
        scale = configs.c_float(192 ** -0.5)
        call = lambda: ops.mla_decode(query, paged, table, dl, scale, splits=8, workspace=workspace, out=out, lse=lse)
    elif args.workload == "absorbed":
        tokens, h = args.seq, args.heads
        ql, qr = randn((1, tokens, h, 512), 0.25), randn((1, tokens, h, 64), 0.25)
        latent, kr = randn((1, tokens, 512), 0.25), randn((1, tokens, 64), 0.25)
        dout = randn((1, tokens, h, 512), 0.2)
        out = torch.empty(1, tokens, h, 512, device=device, dtype=torch.bfloat16)
        lse = torch.empty(1, h, tokens, device=device)
        scale = configs.c_float(576 ** -0.5)
        grads = tuple(torch.empty_like(x) for x in (ql, qr, latent, kr))

        def call():
            ops.mla_forward(ql, qr, latent, kr, scale, out, lse)
            ops.mla_backward(dout, out, lse, ql, qr, latent, kr, scale, grads)
    elif args.workload == "projection":
        tokens, h = args.seq, args.heads
        wkv_b = randn((h, 256, 512), 0.06)
        q_nope, o_latent = randn((1, tokens, h, 128), 0.5), randn((1, tokens, h, 512), 0.5)
        q_latent = torch.empty(1, tokens, h, 512, device=device, dtype=torch.bfloat16)
        o = torch.empty(1, tokens, h, 128, device=device, dtype=torch.bfloat16)

        def call():
            ops.mla_absorb_query(q_nope, wkv_b[:, :128], out=q_latent)
            ops.mla_unabsorb_output(o_latent, wkv_b[:, 128:], out=o)
    elif args.workload == "flash":
        q, k, v = randn((1, 512, 8, 64), 1.0), randn((1, 512, 8, 64), 1.0), randn((1, 512, 8, 64), 1.0)
        out, lse = torch.empty_like(q), torch.empty(1, 8, 512, device=device)
        call = lambda: ops.flash_forward(q, k, v, 0.125, out, lse)
    else:
        source = torch.empty(1 << 28, device=device, dtype=torch.float32).normal_()
        target = torch.empty_like(source)
        call = lambda: target.copy_(source)

    call()
    torch.cuda.synchronize()
    for _ in range(args.steps):
        call()
    torch.cuda.synchronize()
    print(f"{args.workload}: {args.steps} profiled calls done", flush=True)


if __name__ == "__main__":
    main()
