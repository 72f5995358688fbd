"""The other workloads of the headline metric, timed beside the forward one by
``bench.py``: backward TFLOP/s, decode GB/s and the flash-attention forward
time.  All inputs are resident in HBM before the timed region."""

from __future__ import annotations

PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0


def measure(device, event_time_ms, q, k, v, scale, out, lse, steps=40, warmup=15):
    """q, k, v: the S=4096 H=128 prefill inputs already on `device`; out / lse: the
    forward's results for them (the backward's saved tensors)."""
    import torch

    from . import configs, ops

    results = {}
    batch, seq, heads, dqk = q.shape
    dv = v.shape[-1]

    # MLA backward, same shape, dO ~ N(0,1) seed 2
    dout = configs.mla_prefill_dout(batch, seq, heads, dv, seed=2).to(device)
    grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    workspace = ops.mla_prefill_backward_workspace(batch, seq, heads, dqk, dv, device)
    ms, _ = event_time_ms(lambda: ops.mla_prefill_backward(dout, out, lse, q, k, v, scale, workspace, grads),
                          steps, warmup)
    flops = configs.backward_flops(batch, heads, seq, dqk, dv)
    results["mla_backward_S4096_H128"] = {
        "ms": ms, "tflops": flops / ms / 1e9, "frac_of_bf16_peak": flops / ms / 1e9 / PEAK_BF16_TFLOPS,
        "flops": flops, "kernels": "attention_backward_statistics + attention_key_value_gradient + attention_query_gradient"}
    del dout, grads, workspace

    # absorbed decode, B=64 H=128, lengths ~ U[1024,8192] seed 3, 64-token pages
    data = configs.mla_decode_inputs()
    lengths = data["lengths"]
    total = int(lengths.sum())
    dq = data["query"].to(device)
    paged = data["paged"].to(device)
    table = data["table"].to(device)
    dl = lengths.to(device)
    b, h = dq.shape[0], dq.shape[2]
    workspace = ops.mla_decode_workspace(b, h, 8, 512, device)
    dout_o = torch.empty(b, 1, h, 512, device=device, dtype=torch.bfloat16)
    dlse = torch.empty(b, h, 1, device=device, dtype=torch.float32)
    ms, _ = event_time_ms(lambda: ops.mla_decode(dq, paged, table, dl, data["scale"], splits=8, workspace=workspace,
                                                 out=dout_o, lse=dlse), 5 * steps, 3 * warmup)
    nbytes = configs.decode_bytes(total, b, h)
    results["mla_decode_B64_H128"] = {
        "us": ms * 1000.0, "gbs": nbytes / ms / 1e6, "frac_of_hbm_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS,
        "bytes": nbytes, "total_tokens": total, "tflops": configs.decode_flops(total, h) / ms / 1e9,
        "kernels": "mla_decode_split (plans for itself up to 256 sequences) + mla_decode_merge"}
    del paged, workspace

    # long context: MLA prefill forward + backward, B=1 S=16384 H=128.  Timing does not depend on the
    # values, so the inputs are drawn on the GPU (the seeded CPU inputs are what the parity test uses).
    generator = torch.Generator(device=device).manual_seed(4)
    long_seq = 16384
    draw = lambda shape, factor: (torch.randn(shape, device=device, generator=generator) * factor).bfloat16()
    lq, lk = draw((1, long_seq, heads, dqk), 0.5), draw((1, long_seq, heads, dqk), 0.5)
    lv, ldo = draw((1, long_seq, heads, dv), 0.5), draw((1, long_seq, heads, dv), 1.0)
    lout = torch.empty(1, long_seq, heads, dv, device=device, dtype=torch.bfloat16)
    llse = torch.empty(1, heads, long_seq, device=device, dtype=torch.float32)
    ms, _ = event_time_ms(lambda: ops.mla_prefill_forward(lq, lk, lv, scale, lout, llse), 12, 3)
    flops = configs.forward_flops(1, heads, long_seq, dqk, dv)
    results["mla_forward_S16384_H128"] = {"ms": ms, "tflops": flops / ms / 1e9,
                                          "frac_of_bf16_peak": flops / ms / 1e9 / PEAK_BF16_TFLOPS, "flops": flops,
                                          "data": "synthetic, GPU generator"}
    grads = (torch.empty_like(lq), torch.empty_like(lk), torch.empty_like(lv))
    workspace = ops.mla_prefill_backward_workspace(1, long_seq, heads, dqk, dv, device)
    ms, _ = event_time_ms(lambda: ops.mla_prefill_backward(ldo, lout, llse, lq, lk, lv, scale, workspace, grads), 10, 2)
    flops = configs.backward_flops(1, heads, long_seq, dqk, dv)
    results["mla_backward_S16384_H128"] = {"ms": ms, "tflops": flops / ms / 1e9,
                                           "frac_of_bf16_peak": flops / ms / 1e9 / PEAK_BF16_TFLOPS, "flops": flops,
                                           "workspace_gib": workspace.numel() * 4 / 2 ** 30,
                                           "data": "synthetic, GPU generator"}
    del lq, lk, lv, ldo, lout, llse, grads, workspace

    # the reference's own prefill API (absorbed form: 576-wide scores against one shared latent head, 512-wide
    # output), forward and backward, at the sequence length and head count of the headline workload
    try:
        tokens = 4096
        ql, qr = draw((1, tokens, heads, 512), 0.25), draw((1, tokens, heads, 64), 0.25)
        latent, kr = draw((1, tokens, 512), 0.25), draw((1, tokens, 64), 0.25)
        dout_a = draw((1, tokens, heads, 512), 0.2)
        aout = torch.empty(1, tokens, heads, 512, device=device, dtype=torch.bfloat16)
        alse = torch.empty(1, heads, tokens, device=device, dtype=torch.float32)
        ascale = configs.c_float(576 ** -0.5)
        ms, _ = event_time_ms(lambda: ops.mla_forward(ql, qr, latent, kr, ascale, aout, alse), 10, 3)
        pairs = heads * tokens * tokens / 2
        flops = pairs * 2 * (576 + 512)
        results["mla_absorbed_forward_T4096_H128"] = {"ms": ms, "tflops": flops / ms / 1e9,
                                                      "frac_of_bf16_peak": flops / ms / 1e9 / PEAK_BF16_TFLOPS, "flops": flops,
                                                      "entry": "dscuda_mla_forward", "data": "synthetic, GPU generator"}
        agrads = tuple(torch.empty_like(x) for x in (ql, qr, latent, kr))
        ms, _ = event_time_ms(lambda: ops.mla_backward(dout_a, aout, alse, ql, qr, latent, kr, ascale, agrads), 5, 2)
        flops = pairs * 2 * (3 * 576 + 2 * 512)   # S, dP, dV (512), dQ and dK (576): the five products
        results["mla_absorbed_backward_T4096_H128"] = {"ms": ms, "tflops": flops / ms / 1e9,
                                                       "frac_of_bf16_peak": flops / ms / 1e9 / PEAK_BF16_TFLOPS, "flops": flops,
                                                       "entry": "dscuda_mla_backward", "data": "synthetic, GPU generator"}
        del ql, qr, latent, kr, dout_a, aout, alse, agrads
    except Exception as error:
        results["mla_absorbed_T4096_H128"] = {"error": str(error)}

    # the projections either side of the absorbed kernels, 4096 tokens x 128 heads: memory-bound by design
    # (x and y rows once, the head's 128 KB weight from L2), so the rate is bytes of x + y + w over time
    try:
        tokens = 4096
        nope = draw((tokens, heads, 128), 0.5)
        weight = draw((heads, 128, 512), 0.05)
        latent_rows = torch.empty(tokens, heads, 512, device=device, dtype=torch.bfloat16)
        back = torch.empty(tokens, heads, 128, device=device, dtype=torch.bfloat16)
        moved = (nope.numel() + latent_rows.numel() + weight.numel()) * 2
        ms, _ = event_time_ms(lambda: ops.mla_absorb_query(nope, weight, latent_rows), 40, 10)
        results["mla_absorb_query_T4096_H128"] = {"us": ms * 1000.0, "gbs": moved / ms / 1e6, "bytes": moved,
                                                  "frac_of_hbm_peak": moved / ms / 1e6 / PEAK_HBM_GBS,
                                                  "entry": "dscuda_mla_absorb_query"}
        ms, _ = event_time_ms(lambda: ops.mla_unabsorb_output(latent_rows, weight, back), 40, 10)
        results["mla_unabsorb_output_T4096_H128"] = {"us": ms * 1000.0, "gbs": moved / ms / 1e6, "bytes": moved,
                                                     "frac_of_hbm_peak": moved / ms / 1e6 / PEAK_HBM_GBS,
                                                     "entry": "dscuda_mla_unabsorb_output"}
        del nope, weight, latent_rows, back
    except Exception as error:
        results["mla_projection_T4096_H128"] = {"error": str(error)}

    # for scale only: what the vendor's bf16 GEMM (torch.matmul -> hipBLASLt) sustains on this chip with random
    # operands, timed the same way; a plain GEMM is the practical ceiling of any MFMA-bound kernel here
    try:
        size = 8192
        left = draw((size, size), 0.5)
        right = draw((size, size), 0.5)
        product = torch.empty(size, size, device=device, dtype=torch.bfloat16)
        ms, _ = event_time_ms(lambda: torch.matmul(left, right, out=product), 40, 10)
        results["bf16_gemm_8192_for_scale"] = {"ms": ms, "tflops": 2.0 * size ** 3 / ms / 1e9,
                                               "frac_of_bf16_peak": 2.0 * size ** 3 / ms / 1e9 / PEAK_BF16_TFLOPS,
                                               "what": "torch.matmul bf16, 0.5*N(0,1) operands"}
        del left, right, product
    except Exception as error:   # the comparison is optional; never let it break the measurement
        results["bf16_gemm_8192_for_scale"] = {"error": str(error)}

    # flash attention forward, B=1 H=8 S=512 D=64 (latency bound: report time)
    fq, fk, fv, fscale = configs.flash_forward_inputs()
    fq, fk, fv = fq.to(device), fk.to(device), fv.to(device)
    fo, fl = torch.empty_like(fq), torch.empty(1, 8, 512, device=device)
    ms, _ = event_time_ms(lambda: ops.flash_forward(fq, fk, fv, fscale, fo, fl), 200, 50)
    results["flash_forward_B1_H8_S512_D64"] = {"us": ms * 1000.0,
                                               "tflops": configs.forward_flops(1, 8, 512, 64, 64) / ms / 1e9}
    return results
