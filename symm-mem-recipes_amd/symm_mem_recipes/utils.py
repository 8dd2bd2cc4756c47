"""Timing harness with the reference's two entry points
(symm_mem_recipes/utils.py:10-82 ``benchmark_with_profiler``, :85-134
``benchmark_with_event``): warm-up, optional cache flush before every timed call,
median latency in microseconds.

One process drives the GPU here, so there is no rank barrier before the timed
region and ``profile_ranks`` only decides whether this process reports (rank 0
does).  The flush buffer is 1 GiB: the part's last-level cache is 256 MiB, where
the reference flushes 256 MB for a 50 MB L2.
"""
from __future__ import annotations

import re
import statistics
from typing import Callable, List, Optional

import torch

from .symm_mem import get_rank

#: bytes written before a timed call when ``flush_l2`` is set
FLUSH_BYTES = 1 << 30

_spin_cycles_per_ms: Optional[float] = None


def _cycles_per_ms() -> float:
    """Cycles of ``torch.cuda._sleep`` that last one millisecond, measured once."""
    global _spin_cycles_per_ms
    if _spin_cycles_per_ms is None:
        torch.cuda._sleep(1_000_000)
        torch.cuda.synchronize()
        begin = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        begin.record()
        torch.cuda._sleep(10_000_000)
        end.record()
        torch.cuda.synchronize()
        _spin_cycles_per_ms = 10_000_000 / begin.elapsed_time(end)
    return _spin_cycles_per_ms


def _flush_buffer(flush_l2: bool) -> Optional[torch.Tensor]:
    return torch.empty(FLUSH_BYTES // 4, dtype=torch.int32, device="cuda") if flush_l2 else None


def benchmark_with_event(target_fn: Callable[[], None], warmup_iters: int = 200,
                         benchmark_iters: int = 25, profile_ranks: Optional[List[int]] = None,
                         flush_l2: bool = False) -> float:
    """Median latency of ``target_fn`` in microseconds between a pair of stream
    events around every call."""
    cache = _flush_buffer(flush_l2)
    for _ in range(warmup_iters):
        target_fn()
    torch.cuda.synchronize()

    begins = [torch.cuda.Event(enable_timing=True) for _ in range(benchmark_iters)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(benchmark_iters)]
    for begin, end in zip(begins, ends):
        if cache is not None:
            cache.zero_()
        begin.record()
        target_fn()
        end.record()
    torch.cuda.synchronize()
    if get_rank() not in (profile_ranks or [0]):
        return 0
    return statistics.median(b.elapsed_time(e) for b, e in zip(begins, ends)) * 1000


def benchmark_with_profiler(target_fn: Callable[[], None], event_key_regex: str,
                            warmup_iters: int = 200, benchmark_iters: int = 25,
                            profile_ranks: Optional[List[int]] = None,
                            flush_l2: bool = False) -> float:
    """Median device time, in microseconds, of the profiler events whose key
    ``event_key_regex`` matches (``re.match``: anchored at the start of the kernel's
    name), over ``benchmark_iters`` calls of ``target_fn``.  0 when nothing matches."""
    cache = _flush_buffer(flush_l2)
    for _ in range(warmup_iters):
        target_fn()
    torch.cuda.synchronize()

    prof = torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CPU,
                                              torch.profiler.ProfilerActivity.CUDA])
    with prof:
        # keep the device busy while the calls queue up, so that launch gaps are not timed
        torch.cuda._sleep(int(10 * _cycles_per_ms()))
        for _ in range(benchmark_iters):
            if cache is not None:
                cache.zero_()
            target_fn()
        torch.cuda.synchronize()
    if get_rank() not in (profile_ranks or [0]):
        return 0

    pattern = re.compile(event_key_regex)
    latencies_us = [event.device_time for event in prof.events() if pattern.match(event.key)]
    if not latencies_us:
        return 0
    return statistics.median(latencies_us)
