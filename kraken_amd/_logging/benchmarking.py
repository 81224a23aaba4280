"""Event-based latency measurement (method of ``kraken/_logging/benchmarking.py:91-163``)."""
from __future__ import annotations

import inspect
import os
import re
from typing import Callable

import torch


def _takes_index(fn) -> bool:
    try:
        return len(inspect.signature(fn).parameters) >= 1
    except (TypeError, ValueError):
        return False


def benchmark_with_event(
    target_fn: Callable[..., None],
    warmup_iters: int = 20,
    benchmark_iters: int = 25,
    flush_cache: bool = True,
    flush_bytes: int = 1 << 30,
    return_all: bool = False,
    *,
    profile_ranks: list[int] | None = None,
    flush_l2: bool | None = None,
    cuda_graph: bool = False,
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
    The reference's keywords are accepted: ``flush_l2`` (same switch as
    ``flush_cache``), ``cuda_graph`` (``:99-108``: the call is captured once and
    the replays are timed) and ``profile_ranks`` (ignored: one rank).
    ``target_fn`` may also take no argument, as in the reference.
    """
    if "BENCHMARK_ITERS" in os.environ:
        benchmark_iters = int(os.environ["BENCHMARK_ITERS"])
    if flush_l2 is not None:
        flush_cache = flush_l2
    if not _takes_index(target_fn):
        plain_fn = target_fn
        target_fn = lambda i: plain_fn()   # noqa: E731
    if cuda_graph:
        eager_fn = target_fn
        eager_fn(0)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                eager_fn(0)
        torch.cuda.current_stream().wait_stream(side)
        target_fn = lambda i: graph.replay()   # noqa: E731
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


def benchmark_with_profiler(
    target_fn: Callable[[], None],
    event_key_regex: str,
    warmup_iters: int = 20,
    benchmark_iters: int = 100,
    profile_ranks: list[int] | None = None,
    flush_l2: bool = False,
    flush_bytes: int = 1 << 30,
) -> float:
    """Median device time, in microseconds, of the profiler events whose key matches
    ``event_key_regex`` (a kernel name), over ``benchmark_iters`` calls of ``target_fn``.

    Counterpart of ``benchmark_with_profiler`` (``kraken/_logging/benchmarking.py:10-88``):
    warm-up, then the calls under ``torch.profiler`` (CPU + device activities), the
    caches flushed before each call when ``flush_l2`` is set, and the median of the
    matching events' device times (``:78-88``); 0 when nothing matches.  Unlike the
    event method this times the kernels themselves, without the launch gaps.
    """
    if "BENCHMARK_ITERS" in os.environ:
        benchmark_iters = int(os.environ["BENCHMARK_ITERS"])
    cache = torch.empty(flush_bytes // 4, dtype=torch.int32, device="cuda") if flush_l2 else None
    for _ in range(warmup_iters):
        target_fn()
    torch.cuda.synchronize()
    activities = [torch.profiler.ProfilerActivity.CPU, torch.profiler.ProfilerActivity.CUDA]
    with torch.profiler.profile(activities=activities) as prof:
        for _ in range(benchmark_iters):
            if cache is not None:
                cache.zero_()
            target_fn()
        torch.cuda.synchronize()
    pattern = re.compile(event_key_regex)
    lat_us = [ev.device_time for ev in prof.events() if pattern.match(ev.key) and ev.device_time > 0]
    if not lat_us:
        return 0.0
    return float(torch.tensor(lat_us, dtype=torch.float64).median().item())

