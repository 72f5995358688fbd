"""Timing by HIP graph replay.

The reference times every operation from inside a captured graph (``benchmarks/common.py:68-111``): launch overhead
of the Python layer is paid once at capture, and what is measured is the device executing `count` calls back to back.
This module does the same measurement with its own moving parts:

* ``CapturedCalls``   `count` consecutive calls of one backend recorded into a graph on the current stream;
* ``Settings``        the knobs of the command line (calls per graph, warm-up and sample lengths, trials);
* ``time_backends``   calibrates how many replays make one sample, warms the chip up for a set amount of *device*
                      time, then takes the samples, starting each trial with a different backend so that none
                      always runs right after an idle gap or right after the other.

Every sample is the mean time of one call in microseconds.  Outputs are verified once on the first replay and once
after the last, through the ``verify`` callback, so a kernel that breaks only under replay cannot pass unnoticed.
"""

from __future__ import annotations

import math
from dataclasses import dataclass


@dataclass(frozen=True)
class Settings:
    calls_per_graph: int = 10
    warmup_ms: float = 1000.0
    sample_ms: float = 20.0
    trials: int = 9

    def __post_init__(self):
        if self.calls_per_graph < 1 or self.trials < 1 or self.sample_ms <= 0 or self.warmup_ms < 0:
            raise ValueError("calls per graph and trials must be at least 1, the sample length positive")


MOST_REPLAYS = 100000   # per sample, whatever the clock says about a single replay


def replays_per_sample(sample_ms: float, replay_ms: float) -> int:
    """Replays that fill one sample of `sample_ms`: at least one, and a bounded number when the measured replay time
    is zero or absurdly small."""
    if replay_ms * MOST_REPLAYS <= sample_ms:
        return MOST_REPLAYS
    return max(1, math.ceil(sample_ms / replay_ms))


def starting_orders(names, trials: int):
    """For each trial, the backends in the order they are sampled: the list rotated by one more place each time."""
    names = list(names)
    return [names[trial % len(names):] + names[:trial % len(names)] for trial in range(trials)]


class CapturedCalls:
    def __init__(self, call, count: int):
        import torch
        self.count = count
        call()
        call()                       # one-time set-up (function attributes, lazy buffers) happens outside the capture
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=torch.cuda.current_stream()):
            for _ in range(count):
                self.outputs = call()

    def replay(self, times: int = 1) -> None:
        for _ in range(times):
            self.graph.replay()


def _device_ms(events, work) -> float:
    import torch
    begin, end = events
    begin.record()
    work()
    end.record()
    end.synchronize()
    return begin.elapsed_time(end)


def time_backends(backends: dict, settings: Settings, verify=None) -> dict:
    """backend name -> list of `settings.trials` samples (microseconds per call)."""
    import torch
    with torch.no_grad():
        captured = {name: CapturedCalls(call, settings.calls_per_graph) for name, call in backends.items()}
        events = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
        replay_ms = {}
        for name, calls in captured.items():
            calls.replay()
            torch.cuda.synchronize()
            if verify:
                verify(name, calls.outputs)
            replay_ms[name] = min(_device_ms(events, calls.replay) for _ in range(2))
        per_round = sum(replay_ms.values())
        rounds = math.ceil(settings.warmup_ms / per_round) if per_round > 0 else 0
        for _ in range(rounds):
            for calls in captured.values():
                calls.replay()
        torch.cuda.synchronize()
        # the chip is warm now: the replay time that sizes the samples is measured again
        repeats = {name: replays_per_sample(settings.sample_ms, _device_ms(events, calls.replay))
                   for name, calls in captured.items()}
        samples = {name: [] for name in captured}
        for order in starting_orders(captured, settings.trials):
            for name in order:
                calls = captured[name]
                elapsed = _device_ms(events, lambda: calls.replay(repeats[name]))
                samples[name].append(1000.0 * elapsed / (repeats[name] * calls.count))
        if verify:
            for name, calls in captured.items():
                verify(name, calls.outputs)
    return samples
