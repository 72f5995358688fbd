"""Headline benchmark: one MI355X, synthetic DeepSeek-V3-shaped inputs.

``python bench.py --gpus 1 --steps K --warmup W`` prints one JSON line.  A step
is one MLA prefill forward over the S=4096, H=128, 192/192/128 workload with
all inputs resident in HBM; ``value`` is its algorithmic TFLOP/s (causal pair
count S^2/2).  The ``roofline`` object prices the forward kernel against the
chip's dense bf16 MFMA peak from its own event-timed launches, ``extra`` holds
the other workloads of the metric (backward TFLOP/s, decode GB/s, flash
forward time), and ``cpu_baseline`` is the fp32 CPU oracle timed on this
machine's host cores over a sample of heads of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

PROFILES = ROOT / "profiles"


def profiled_figures(stem, kernel_prefix):
    """(HBM bytes per launch, settled microseconds) of the first kernel whose name starts with `kernel_prefix` in
    profiles/<stem>.md, the summary `python -m dscuda_amd.profiler.capture` writes from rocprofv3's FETCH_SIZE /
    WRITE_SIZE passes (each scaled by what the same counter reads for a 1 GiB device copy) and its kernel trace.
    A recorded measurement of the committed kernels, not something this script can observe; (None, None) if the
    summary is missing."""
    path = PROFILES / f"{stem}.md"
    if not path.is_file():
        return None, None
    for line in path.read_text().splitlines():
        line = line.strip()
        if line.startswith(kernel_prefix) and " :: time_us = " in line:   # not the counter lines of the same kernel
            fields = dict(part.strip().split(" = ") for part in line.split(" :: ", 1)[1].split(" ; "))
            nbytes = float(fields.get("fabric_bytes", fields.get("hbm_bytes", "nan")))
            return (None if nbytes != nbytes else nbytes), float(fields["time_us"])
    return None, None


SETTLE_MS = 40.0   # back-to-back launches before any timing: the chip's clock needs ~25 ms of load to settle


def event_time_ms(function, steps, warmup, settle_ms=SETTLE_MS):
    """Average duration of `function` over `steps` launches, from events on torch's
    current stream (the stream the kernels are enqueued on).  Before the `warmup`
    untimed launches the function is run back to back for `settle_ms` of wall time,
    so that a small `warmup` still times the kernel at the clock a loaded chip runs at."""
    import torch
    deadline = time.perf_counter() + settle_ms / 1000.0
    while time.perf_counter() < deadline:
        for _ in range(8):
            function()
        torch.cuda.synchronize()
    for _ in range(warmup):
        function()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    wall = time.perf_counter()
    start.record()
    for _ in range(steps):
        function()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - wall) * 1000.0
    return start.elapsed_time(stop) / steps, wall / steps


def cpu_baseline_forward(q, k, v, scale, gpu_out, gpu_lse, sample_heads):
    """fp32 oracle on the host cores over `sample_heads` heads; also checks the
    GPU result of the same heads.  Only this leg touches oracle/."""
    import torch
    from dscuda_amd.harness import configs
    from oracle import attention_oracle as oracle

    heads = list(range(0, q.shape[2], max(1, q.shape[2] // sample_heads)))[:sample_heads]
    oracle.causal_attention_forward(q[:, :256], k[:, :256], v[:, :256], scale, heads=heads[:1])  # warm threads
    begin = time.perf_counter()
    expected, expected_lse = oracle.causal_attention_forward(q, k, v, scale, heads=heads)
    seconds = time.perf_counter() - begin
    flops = configs.forward_flops(q.shape[0], len(heads), q.shape[1], q.shape[3], v.shape[3])
    worst, mean = oracle.error_stats(gpu_out[:, :, heads].float().cpu(), expected)
    lse_err = (gpu_lse[:, heads].cpu() - expected_lse).abs().max().item()
    baseline = {
        "value": flops / seconds / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"{len(heads)} of {q.shape[2]} heads of the same workload, unfused fp32 PyTorch oracle, "
                  f"{seconds:.1f} s, {torch.get_num_threads()} intra-op threads (the cores counted), "
                  f"os.cpu_count()={os.cpu_count()}, torch {torch.__version__}",
    }
    parity = {"heads_checked": len(heads), "o_max_abs": worst, "o_mean_abs": mean, "lse_max_abs": lse_err,
              "ok": bool(worst <= 2e-2 and mean <= 2e-3 and lse_err <= 1e-3)}
    return baseline, parity


def cpu_baselines_of_the_other_legs(q, k, v, scale, gpu_out, gpu_lse, backward_heads=8):
    """The fp32 oracle timed on the host cores for the backward (a sample of heads of the S=4096 workload) and the
    decode (all 64 sequences of the B=64 workload): reported beside the GPU figures of `extra`, never a target."""
    import torch
    from dscuda_amd.harness import configs
    from oracle import attention_oracle as oracle

    results = {}
    batch, seq, heads, dqk = q.shape
    dv = v.shape[-1]
    sample = list(range(0, heads, max(1, heads // backward_heads)))[:backward_heads]
    dout = configs.mla_prefill_dout(batch, seq, heads, dv, seed=2)
    sub = lambda t: t[:, :, sample]
    saved_out, saved_lse = gpu_out[:, :, sample].cpu(), gpu_lse[:, sample].cpu()
    begin = time.perf_counter()
    oracle.attention_backward(sub(dout), saved_out, saved_lse, sub(q), sub(k), sub(v), scale)
    seconds = time.perf_counter() - begin
    flops = configs.backward_flops(batch, len(sample), seq, dqk, dv)
    results["cpu_baseline_mla_backward_S4096"] = {
        "value": flops / seconds / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"{len(sample)} of {heads} heads, analytic fp32 backward of the oracle, {seconds:.1f} s"}

    data = configs.mla_decode_inputs()
    lengths = data["lengths"]
    repeats, seconds = 0, 0.0
    begin = time.perf_counter()
    while seconds < 5.0:   # the whole batch takes a fraction of a second: repeat it for a sample worth timing
        for b in range(lengths.numel()):
            n = int(lengths[b])
            oracle.mla_decode_unrounded(data["query"][b:b + 1], data["cache"][b:b + 1, :n], lengths[b:b + 1], data["scale"])
        repeats += 1
        seconds = time.perf_counter() - begin
    seconds /= repeats
    nbytes = configs.decode_bytes(int(lengths.sum()), lengths.numel(), data["query"].shape[2])
    results["cpu_baseline_mla_decode_B64_H128"] = {
        "value": nbytes / seconds / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"all {lengths.numel()} sequences, fp32 oracle one sequence at a time, {repeats} passes of "
                  f"{seconds:.2f} s each"}
    return results


def main():
    parser = argparse.ArgumentParser(description=__doc__)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=50)
    parser.add_argument("--cpu-heads", type=int, default=128, help="heads in the CPU baseline sample")
    parser.add_argument("--no-extra", action="store_true", help="skip the backward / decode / flash measurements")
    args = parser.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (the workload shards over heads "
                 "without communication); run with --gpus 1")

    import torch
    from dscuda_amd.harness import configs, ops

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    device = torch.device("cuda:0")

    # ---- headline: MLA prefill forward, S=4096, H=128, 192/192/128, seed 1 + RoPE
    batch, seq, heads, dqk, dv = 1, 4096, 128, 192, 128
    q, k, v, scale = configs.mla_prefill_inputs(batch, seq, heads, seed=1)
    dq, dk, dvv = q.to(device), k.to(device), v.to(device)
    out = torch.empty(batch, seq, heads, dv, device=device, dtype=torch.bfloat16)
    lse = torch.empty(batch, heads, seq, device=device, dtype=torch.float32)

    def forward_step():
        ops.mla_prefill_forward(dq, dk, dvv, scale, out, lse)

    kernel_ms, wall_ms = event_time_ms(forward_step, args.steps, args.warmup)
    flops = configs.forward_flops(batch, heads, seq, dqk, dv)
    achieved = flops / kernel_ms / 1e9

    extra = {}
    if not args.no_extra:
        from dscuda_amd.harness import extra_workloads
        extra = extra_workloads.measure(device, event_time_ms, dq, dk, dvv, scale, out, lse)

    baseline, parity = cpu_baseline_forward(q, k, v, scale, out, lse, args.cpu_heads)
    if not args.no_extra:
        extra.update(cpu_baselines_of_the_other_legs(q, k, v, scale, out, lse))
    traffic, profiled_us = profiled_figures("mla_prefill_forward_S4096_H128", "attention_forward_pingpong_kernel")

    line = {
        "metric": "MLA fwd/bwd TFLOP/s (% bf16 MFMA peak); decode HBM GB/s, 1xMI355X",
        "value": flops / wall_ms / 1e9,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": SETTLE_MS,
        "ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "MLA prefill forward, B=1 S=4096 H=128, d_qk=128+64, d_v=128, causal, "
                               "0.5*N(0,1) seed 1, RoPE theta=10000, scale 1/sqrt(192)"},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": traffic,
                     "traffic_source": "profiles/mla_prefill_forward_S4096_H128.md (rocprofv3 FETCH_SIZE + WRITE_SIZE: bytes between the L2s and the fabric, an upper bound of the HBM bytes since the Infinity Cache serves part of them)",
                     "kernel": "attention_forward_pingpong_kernel<192,128>", "kernel_ms": kernel_ms,
                     "profiled_kernel_ms": None if profiled_us is None else profiled_us / 1000.0,
                     "flops_per_launch": flops},
        "cpu_baseline": baseline,
        "parity": parity,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
