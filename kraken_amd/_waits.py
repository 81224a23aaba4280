"""Bounded device-side waits must not fail silently.

The flag waits of the overlap paths (tiles that wait for their rows, copies that wait for their
band, wavefronts of a split row that wait for each other) give up after a limit and record that
in an int32 ``status`` word on the device, so that kernels and streams always drain where the
reference would block for ever (``kraken/fused/all_gather_matmul.py:95-110``,
``gemm_reduce_scatter_ce_persistent.py:153-163``).  A caller who passes a ``status`` tensor reads
it themselves.  When none is passed, the wrappers take the word this module keeps for the
(device, stream) they run on and register it behind the work: the word is mirrored into pinned
host memory by a copy that is ordered behind the work, and the mirror is read -- without any
synchronisation -- once an event behind that copy has completed: on a later call of any of these
functions or on ``check()``.  A non-zero word raises, naming every call whose result is invalid.

The word of a stream is sticky: after a wait has run out, the waits of the calls already enqueued
behind it on the same stream see it and give up at once instead of each running to the limit
(their results are invalid too and are reported together); the word is cleared, in stream order,
when the failure is reported.
"""
from __future__ import annotations

import threading
import time

import torch

from ._lib import KrakenAmdError

_lock = threading.Lock()
# (event behind the mirror copy, pinned host mirror, device word, what, the stream the work is on)
_pending: list[tuple[torch.cuda.Event, torch.Tensor, torch.Tensor, str, torch.cuda.Stream]] = []
_words: dict[tuple[int, int], torch.Tensor] = {}
_free_mirrors: list[torch.Tensor] = []
_last_watch: dict[int, float] = {}       # id of a status word -> time of its last mirror copy
_failure_hooks: list = []


def on_failure(hook) -> None:
    """Register a function to be called (no arguments) when a failed wait is about to be raised."""
    _failure_hooks.append(hook)


def new_status(dev: torch.device) -> torch.Tensor:
    """The status word of the current stream of ``dev`` (zero unless an earlier wait on this stream
    has run out and has not been reported yet).  Every wait of one call shares it: the first wait
    that runs out makes the later ones give up at once instead of each running to the limit."""
    key = (dev.index if dev.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(dev).cuda_stream)
    with _lock:
        word = _words.get(key)
        if word is None:
            word = torch.zeros(1, dtype=torch.int32, device=dev)
            _words[key] = word
    return word


def watch(status: torch.Tensor, what: str, min_interval_s: float = 0.0) -> None:
    """Register ``status`` to be read once everything enqueued so far on the current stream is done.
    ``min_interval_s`` > 0: skip the registration if this word was registered less than that long
    ago (for calls of a few microseconds; the word is sticky, so a later look still finds a failure)."""
    if torch.cuda.is_current_stream_capturing():
        return          # a captured call cannot be read back here; its caller passes a status of its own
    if min_interval_s > 0.0:
        now = time.monotonic()
        with _lock:
            if now - _last_watch.get(id(status), -1e30) < min_interval_s:
                return
            _last_watch[id(status)] = now
    with _lock:
        mirror = _free_mirrors.pop() if _free_mirrors else torch.zeros(1, dtype=torch.int32, pin_memory=True)
    mirror.copy_(status, non_blocking=True)          # ordered behind the work on the current stream
    stream = torch.cuda.current_stream(status.device)
    ev = torch.cuda.Event()
    ev.record(stream)
    with _lock:
        _pending.append((ev, mirror, status, what, stream))


def check(block: bool = False) -> None:
    """Raise if a registered wait ran out.  ``block=False`` looks only at work that has finished
    and never synchronises (it reads host memory that a completed copy has filled);
    ``block=True`` waits for all registered work first and then also reads every stream's word
    directly (a synchronising read), so that nothing a rate-limited registration skipped is missed."""
    if torch.cuda.is_current_stream_capturing():
        return
    failed: list[tuple[str, int]] = []
    stuck: list[tuple[torch.Tensor, torch.cuda.Stream]] = []
    with _lock:
        rest = []
        for entry in _pending:
            ev, mirror, status, what, stream = entry
            if block:
                ev.synchronize()
            if not ev.query():
                rest.append(entry)
                continue
            v = int(mirror[0])                       # pinned host memory: no device access
            _free_mirrors.append(mirror)
            if v != 0:
                failed.append((what, v))
                if not any(s is status for s, _ in stuck):
                    stuck.append((status, stream))
        _pending[:] = rest
        words = list(_words.items()) if block else []
    if words:
        torch.cuda.synchronize()
    for (dev_index, stream_handle), word in words:
        v = int(word.item())
        if v != 0 and not any(s is word for s, _ in stuck):
            failed.append((f"a call on stream {stream_handle:#x} of device {dev_index}", v))
            stuck.append((word, torch.cuda.ExternalStream(stream_handle, device=dev_index) if stream_handle else
                          torch.cuda.default_stream(dev_index)))
    if failed:
        for s, stream in stuck:
            with torch.cuda.stream(stream):
                s.zero_()                            # the word starts afresh, in the order of its stream
        for hook in _failure_hooks:
            hook()
        calls = "; ".join(f"{what} (status {v})" for what, v in failed)
        raise KrakenAmdError(
            f"a bounded wait for a progress flag ran out in: {calls}; the results of these calls are invalid")
