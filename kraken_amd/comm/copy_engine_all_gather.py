"""Chunked all-gather with arrival flags (``kraken/comm/copy_engine_all_gather.py``)."""
from __future__ import annotations

import torch

from .. import _lib
from ._common import PeerBuffers

_backend_streams: dict[int, torch.cuda.Stream] = {}


def _get_backend_stream(dev: torch.device) -> torch.cuda.Stream:
    """One side stream per device for the copies (default priority)."""
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    if idx not in _backend_streams:
        _backend_streams[idx] = torch.cuda.Stream(device=dev)
    return _backend_streams[idx]


def _check_progress(progress: torch.Tensor, n: int) -> None:
    assert progress.dtype in (torch.int32, torch.uint32), "progress must be a 32-bit integer tensor"
    assert progress.is_contiguous() and progress.numel() >= n


def _copy_engine_all_gather_w_progress(
    output: torch.Tensor,
    inp,
    progress: torch.Tensor,
    splits_per_rank: int,
    backend_stream: torch.cuda.Stream | None = None,
    *,
    rank: int = 0,
    copy_engine: bool = False,
) -> torch.cuda.Stream:
    """Copy the W shards into ``output`` chunk by chunk on a side stream, flagging each chunk.

    Counterpart of ``_copy_engine_all_gather_w_progress``
    (``kraken/comm/copy_engine_all_gather.py:6-60``).  ``inp`` holds the W
    ranks' shards — the ``[W, m, ...]`` stack or a list of W tensors, standing
    in for the peers' symmetric buffers (``:41-43``).  On the side stream, in
    the reference's order (source ranks ``rank+1, rank+2, ..., rank``, ``:38-39``),
    every one of the ``W * splits_per_rank`` chunks is copied into its place in
    ``output`` and then ``progress[chunk]`` is set to 1 by a stream-ordered
    flag write (``:47-53``).  The side stream first waits for the current
    stream (``:35``); the caller makes the current stream wait for the returned
    stream when it needs the gathered tensor (``:118``).  The copies are ordinary
    device-to-device copy kernels; ``copy_engine=True`` hands them to the GPU's
    copy engines (``kr_copy_engine_memcpy``), which take no compute units but
    are slower within one GPU.  ``progress`` must have been zeroed on the current
    stream beforehand.
    """
    peers = PeerBuffers(inp, dtypes=(torch.bfloat16, torch.float8_e4m3fn))
    W = peers.W
    assert 0 <= rank < W
    assert peers.cap % splits_per_rank == 0
    n_chunks = W * splits_per_rank
    _check_progress(progress, n_chunks)
    out_shape = list(peers.slice(0).shape)
    out_shape[0] *= W
    assert list(output.shape) == out_shape, (list(output.shape), out_shape)
    assert output.is_contiguous() and output.dtype == peers.slice(0).dtype
    dev = _lib.require_device(*peers.tensors, output, progress)
    if backend_stream is None:
        backend_stream = _get_backend_stream(dev)
    lib = _lib.load()
    chunk = peers.cap // splits_per_rank
    flat_out = output.view(-1)
    backend_stream.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(backend_stream):
        for step in range(W):
            src_rank = (rank + step + 1) % W
            src = peers.slice(src_rank).reshape(-1)
            for split_id in range(splits_per_rank):
                c = src_rank * splits_per_rank + split_id
                dst_c, src_c = flat_out[c * chunk:(c + 1) * chunk], src[split_id * chunk:(split_id + 1) * chunk]
                if copy_engine:
                    _lib.copy_engine_copy(dst_c, src_c, backend_stream.cuda_stream)
                else:
                    dst_c.copy_(src_c)
                rc = lib.kr_stream_write_value32(progress.data_ptr() + 4 * c, 1, backend_stream.cuda_stream)
                _lib.check(rc, "stream_write_value32")
    return backend_stream


def all_gather_w_progress(a_shared, a_out: torch.Tensor | None = None, progress: torch.Tensor | None = None,
                          **kwargs) -> torch.Tensor:
    """All-gather of the W shards into one tensor, chunk flags in ``progress``.

    Counterpart of ``all_gather_w_progress``
    (``kraken/comm/copy_engine_all_gather.py:63-120``): allocates ``a_out`` and
    ``progress`` when not given, zeroes ``progress`` (``:108``), runs the chunked
    copy on the side stream and makes the current stream wait for it.  kwargs:
    ``splits_per_rank`` (default 1), ``rank`` (default 0), ``copy_engine`` (default False).
    """
    peers = PeerBuffers(a_shared)
    splits = kwargs.get("splits_per_rank", 1)
    rank = kwargs.get("rank", 0)
    dev = _lib.require_device(*peers.tensors)
    shape = list(peers.slice(0).shape)
    shape[0] *= peers.W
    if a_out is None:
        a_out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
    if progress is None:
        progress = torch.zeros(peers.W * splits, dtype=torch.int32, device=dev)
    else:
        progress.fill_(0)
    stream = _copy_engine_all_gather_w_progress(a_out, a_shared, progress, splits, rank=rank,
                                                copy_engine=kwargs.get("copy_engine", False))
    torch.cuda.current_stream(dev).wait_stream(stream)
    return a_out
