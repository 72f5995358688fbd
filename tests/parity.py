"""Shared tolerance checks for the GPU parity tests.

The bar (bf16 outputs and gradients against the fp32 oracle): max-abs error
<= 2e-2, mean-abs error <= 2e-3, logsumexp within 1e-3.
"""

import sys

import torch

from oracle.attention_oracle import error_stats

MAX_ABS = 2e-2
MEAN_ABS = 2e-3
LSE_ABS = 1e-3


def announce(*parts):
    """Name the case before the GPU step so that a fault can be attributed."""
    print("[case]", *parts, flush=True)
    sys.stdout.flush()


def assert_close_bf16(name, actual, expected, max_abs=MAX_ABS, mean_abs=MEAN_ABS):
    actual = actual.detach().float().cpu()
    expected = expected.detach().float().cpu()
    assert actual.shape == expected.shape, (name, actual.shape, expected.shape)
    assert torch.isfinite(actual).all(), f"{name}: non-finite values"
    worst, mean = error_stats(actual, expected)
    assert worst <= max_abs and mean <= mean_abs, f"{name}: max-abs {worst:.3e} mean-abs {mean:.3e}"
    return worst, mean


def assert_close_lse(name, actual, expected, tol=LSE_ABS):
    actual = actual.detach().float().cpu()
    expected = expected.detach().float().cpu()
    assert actual.shape == expected.shape, (name, actual.shape, expected.shape)
    worst = (actual - expected).abs().max().item()
    assert worst <= tol, f"{name}: max-abs {worst:.3e}"
    return worst
