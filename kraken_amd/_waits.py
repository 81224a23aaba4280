"""Bounded device-side waits must not fail silently.

The flag waits of the overlap paths (tiles that wait for their rows, copies that wait for their
band) give up after a limit and record that in an int32 ``status`` word on the device, so that
kernels and streams always drain where the reference would block for ever
(``kraken/fused/all_gather_matmul.py:95-110``, ``gemm_reduce_scatter_ce_persistent.py:153-163``).
A caller who passes a ``status`` tensor reads it themselves.  When none is passed, the wrappers
take one from here and register it behind the work: it is read as soon as the work is known to
have finished -- on a later call of any of these functions or on ``check()`` -- and a non-zero
word raises, naming the call whose result is invalid.
"""
from __future__ import annotations

import torch

from ._lib import KrakenAmdError

_pending: list[tuple[torch.cuda.Event, torch.Tensor, str]] = []


def new_status(dev: torch.device) -> torch.Tensor:
    """A zeroed status word.  Every wait of one call shares it: the first wait that runs out
    makes the later ones give up at once instead of each running to the limit."""
    return torch.zeros(1, dtype=torch.int32, device=dev)


def watch(status: torch.Tensor, what: str) -> None:
    """Register ``status`` to be read once everything enqueued so far on the current stream is done."""
    if torch.cuda.is_current_stream_capturing():
        return          # a captured call cannot be read back here; its caller passes a status of its own
    ev = torch.cuda.Event()
    ev.record(torch.cuda.current_stream(status.device))
    _pending.append((ev, status, what))


def check(block: bool = False) -> None:
    """Raise if a registered wait ran out.  ``block=False`` looks only at work that has finished
    (no synchronisation); ``block=True`` waits for all of it first."""
    if torch.cuda.is_current_stream_capturing():
        return
    failed = None
    rest = []
    for ev, status, what in _pending:
        if block:
            ev.synchronize()
        if not ev.query():
            rest.append((ev, status, what))
            continue
        v = int(status.item())
        if v != 0 and failed is None:
            failed = (what, v)
    _pending[:] = rest
    if failed is not None:
        raise KrakenAmdError(
            f"{failed[0]}: a bounded wait for a progress flag ran out (status {failed[1]}); "
            "the result of that call is invalid")
