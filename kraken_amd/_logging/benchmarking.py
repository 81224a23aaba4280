"""Event-based latency measurement (method of ``kraken/_logging/benchmarking.py:91-163``)."""
from __future__ import annotations

import os
from typing import Callable

import torch


def benchmark_with_event(
    target_fn: Callable[[int], None],
    warmup_iters: int = 20,
    benchmark_iters: int = 25,
    flush_cache: bool = True,
    flush_bytes: int = 1 << 30,
    return_all: bool = False,
):
    """Median latency of ``target_fn`` in microseconds.

    Same protocol as the reference's ``benchmark_with_event``: untimed warm-up
    calls (``:119-120``), then ``benchmark_iters`` calls each bracketed by its
    own start/end event on the current stream (``:126-129,152-158``), the
    caches defeated before each timed call (``:116-117,153-154``), and the
    median reported (``:160-163``).  Two differences: the flush buffer is 1 GiB
    because the MI355X last-level (Infinity) cache is 256 MB — the size of the
    reference's whole flush buffer — and ``target_fn`` receives the iteration
    index so that callers can rotate through several input sets.
    ``BENCHMARK_ITERS`` overrides the iteration count like in the reference.
    """
    if "BENCHMARK_ITERS" in os.environ:
        benchmark_iters = int(os.environ["BENCHMARK_ITERS"])
    cache = None
    if flush_cache:
        cache = torch.empty(flush_bytes // 4, dtype=torch.int32, device="cuda")
    for i in range(warmup_iters):
        target_fn(i)
    torch.cuda.synchronize()
    begin = [torch.cuda.Event(enable_timing=True) for _ in range(benchmark_iters)]
    end = [torch.cuda.Event(enable_timing=True) for _ in range(benchmark_iters)]
    for i in range(benchmark_iters):
        if cache is not None:
            cache.zero_()
        begin[i].record()
        target_fn(i)
        end[i].record()
    torch.cuda.synchronize()
    lat_us = [b.elapsed_time(e) * 1000.0 for b, e in zip(begin, end)]
    med = float(torch.tensor(lat_us).median().item())
    if return_all:
        return med, lat_us
    return med
