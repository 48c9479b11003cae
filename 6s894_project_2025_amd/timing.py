"""Device-side timing helpers shared by ``bench.py`` and the harness.

All of them time on torch's *current* stream, which is the stream the ops launch on, with
HIP events; nothing here synchronises inside the timed window."""
from __future__ import annotations

import time
from typing import Callable

import torch


def event_window_ms(fn: Callable[[], None], calls: int, warmup: int = 3) -> tuple[float, float]:
    """``warmup`` untimed calls, then ``calls`` back-to-back calls inside one event window (the
    protocol of the reference's bench/bench.py:112-127).  Returns (device ms per call, host
    wall-clock ms per call)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    first = torch.cuda.Event(enable_timing=True)
    last = torch.cuda.Event(enable_timing=True)
    wall0 = time.perf_counter()
    first.record()
    for _ in range(calls):
        fn()
    last.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - wall0) * 1e3
    calls = max(calls, 1)
    return first.elapsed_time(last) / calls, wall_ms / calls


def steady_window_ms(fn: Callable[[], None], calls: int, warm_ms: float = 60.0) -> tuple[float, float]:
    """Like :func:`event_window_ms`, but the untimed warm-up lasts at least ``warm_ms`` of device
    time: matrix-core-bound kernels keep speeding up for the first ~30 ms of sustained load while
    the clocks ramp, so a three-call warm-up would time the ramp rather than the kernel."""
    fn()
    torch.cuda.synchronize()
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    spent, batch = 0.0, 4
    while spent < warm_ms:
        a.record()
        for _ in range(batch):
            fn()
        b.record()
        torch.cuda.synchronize()
        spent += a.elapsed_time(b)
        batch = min(batch * 2, 256)
    return event_window_ms(fn, calls, 0)


def best_single_call_ms(fn: Callable[[], None], runs: int, warmup: int = 2) -> float:
    """Minimum over ``runs`` individually timed calls after ``warmup`` calls (the protocol of
    fused_ht/fusion_pipelined.cu:631-683)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(runs):
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        best = min(best, float(a.elapsed_time(b)))
    return best
