"""The other workloads of the headline metric, timed beside the forward one by
``bench.py``: backward TFLOP/s, decode GB/s and the flash-attention forward
time.  Each entry is skipped (with the reason) while its kernel is missing."""

from __future__ import annotations


def measure(device, event_time_ms, q, k, v, scale, out, lse):
    import torch

    from . import configs, ops

    results = {}

    # flash attention forward, B=1 H=8 S=512 D=64 (latency bound: report time)
    fq, fk, fv, fscale = configs.flash_forward_inputs()
    fq, fk, fv = fq.to(device), fk.to(device), fv.to(device)
    fo, fl = torch.empty_like(fq), torch.empty(1, 8, 512, device=device)
    ms, _ = event_time_ms(lambda: ops.flash_forward(fq, fk, fv, fscale, fo, fl), 50, 10)
    results["flash_forward_B1_H8_S512_D64"] = {"us": ms * 1000.0,
                                               "tflops": configs.forward_flops(1, 8, 512, 64, 64) / ms / 1e9}
    return results
