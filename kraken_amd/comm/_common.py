"""Shared argument handling of the W-way reduce wrappers."""
from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from .. import _lib, _waits


class PeerBuffers:
    """The W buffers a reduce reads: one per rank, all on this GPU.

    Stands in for the peers' symmetric-memory buffers of the reference
    (``symm_mem_hdl.buffer_ptrs_dev``, ``kraken/comm/one_shot_all_reduce.py:96-99``).
    Two forms are accepted wherever the reference takes its symmetric buffer:

    * one ``[W, ...]`` tensor whose slices are the W buffers (slices must be
      contiguous, the stride between them is free) — goes to the stacked entry
      points of the library;
    * a list or tuple of W separately allocated tensors of one shape — goes to
      the pointer-table entry points (``kr_*_ptrs_bf16``), which is also how W
      real peer mappings would be handed over.

    Both forms give bit-identical results: the kernels are the same.
    """

    def __init__(self, buffers: torch.Tensor | Sequence[torch.Tensor], dtypes=(torch.bfloat16,)):
        if isinstance(buffers, torch.Tensor):
            assert buffers.dim() >= 2, "expected a stacked tensor of shape [W, ...]"
            assert buffers.dtype in dtypes, "Only bfloat16 is supported for now."
            self.W = buffers.shape[0]
            assert self.W >= 1
            assert buffers[0].is_contiguous(), "each of the W slices must be contiguous"
            self.cap = buffers[0].numel()
            self.stride = buffers.stride(0) if self.W > 1 else self.cap
            self.stacked = buffers
            self.tensors = [buffers]
        else:
            bufs = list(buffers)
            assert len(bufs) >= 1, "expected W >= 1 buffers"
            for t in bufs:
                assert isinstance(t, torch.Tensor), "expected a tensor or a sequence of tensors"
                assert t.dtype in dtypes and t.dtype == bufs[0].dtype, "Only bfloat16 is supported for now."
                assert t.is_contiguous(), "each of the W buffers must be contiguous"
                assert t.shape == bufs[0].shape, "the W buffers must have one shape"
            self.W = len(bufs)
            self.cap = bufs[0].numel()
            self.stride = None
            self.stacked = None
            self.tensors = bufs

    def slice(self, rank: int) -> torch.Tensor:
        """Buffer of rank ``rank``."""
        return self.stacked[rank] if self.stacked is not None else self.tensors[rank]

    def _table(self, elem_off: int):
        # host array of W device pointers, each moved on by elem_off bf16 elements
        return (ctypes.c_void_p * self.W)(*[t.data_ptr() + 2 * elem_off for t in self.tensors])

    def reduce(self, elem_off, numel, bias_ptr, bias_numel, D, bias_first, out_ptr, stream) -> int:
        """``kr_reduce_bf16`` / ``kr_reduce_ptrs_bf16`` on elements [elem_off, elem_off + numel)."""
        lib = _lib.load()
        if self.stacked is not None:
            return lib.kr_reduce_bf16(self.stacked.data_ptr() + 2 * elem_off, self.W, self.stride, numel,
                                      bias_ptr, bias_numel, D, bias_first, out_ptr, stream)
        return lib.kr_reduce_ptrs_bf16(self._table(elem_off), self.W, numel, bias_ptr, bias_numel, D,
                                       bias_first, out_ptr, stream)

    def reduce_striped(self, numel, bias_ptr, block, rank, out_ptr, stream) -> int:
        lib = _lib.load()
        if self.stacked is not None:
            return lib.kr_reduce_striped_bf16(self.stacked.data_ptr(), self.W, self.stride, numel, bias_ptr,
                                              block, rank, out_ptr, stream)
        return lib.kr_reduce_striped_ptrs_bf16(self._table(0), self.W, numel, bias_ptr, block, rank, out_ptr,
                                               stream)

    def reduce_rmsnorm(self, rows, D, bias_ptr, bias_is_vector, w_ptr, eps, y_ptr, stream) -> int:
        lib = _lib.load()
        dev = self.tensors[0].device
        ws = row_workspace(dev, lib.kr_rmsnorm_workspace_bytes(self.W, rows, D))
        ws_ptr, ws_bytes = (ws.data_ptr(), ws.numel()) if ws is not None else (None, 0)
        # a few long rows: their wavefronts meet in the workspace, a bounded wait that reports through
        # the stream's status word like the flag waits of the overlap paths
        status = _waits.new_status(dev) if ws is not None else None
        if self.stacked is not None:
            rc = lib.kr_reduce_rmsnorm_ws_bf16(self.stacked.data_ptr(), self.W, self.stride, rows, D, bias_ptr,
                                               bias_is_vector, w_ptr, eps, y_ptr, ws_ptr, ws_bytes, _lib.ptr(status),
                                               stream)
        else:
            rc = lib.kr_reduce_rmsnorm_ptrs_ws_bf16(self._table(0), self.W, rows, D, bias_ptr, bias_is_vector,
                                                    w_ptr, eps, y_ptr, ws_ptr, ws_bytes, _lib.ptr(status), stream)
        if status is not None and rc == 0:
            # (the word is sticky and these calls take microseconds: mirroring it to the host now and
            # then is enough to report a time-out, every call would cost more than the kernel)
            _waits.watch(status, "reduce + RMSNorm of a few long rows (rows spread over many compute units)",
                         min_interval_s=0.05)
        return rc


_row_workspaces: dict[tuple[int, int], tuple[torch.Tensor, torch.cuda.Stream]] = {}


def row_workspace(dev: torch.device, nbytes: int) -> torch.Tensor | None:
    """Workspace of the split-row RMSNorm kernel: one zero-initialised buffer per (device, stream
    that is current at the call), so that eager calls on different streams never share one; the
    kernels keep it consistent afterwards.  A call that is captured into a graph bakes in the
    workspace of the capture stream, whatever stream the graph is later replayed on: replays of
    that graph must not overlap each other, other graphs captured on the same stream, or eager
    calls on the capture stream (calls that share a workspace and overlap give NaN rows or wrong
    ones).  After a reported time-out of the rows' exchange every workspace is zeroed again."""
    if nbytes <= 0:
        return None
    stream = torch.cuda.current_stream(dev)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), stream.cuda_stream)
    entry = _row_workspaces.get(key)
    if entry is None or entry[0].numel() < nbytes:
        entry = (torch.zeros(nbytes, dtype=torch.uint8, device=dev), stream)
        _row_workspaces[key] = entry
    return entry[0]


def _zero_row_workspaces() -> None:
    # after a time-out the slots of a workspace may carry tags that a later call would take for fresh ones
    for ws, stream in _row_workspaces.values():
        with torch.cuda.stream(stream):
            ws.zero_()


_waits.on_failure(_zero_row_workspaces)


def check_stack(stacked: torch.Tensor | Sequence[torch.Tensor]) -> PeerBuffers:
    """Validate the W buffers (stacked tensor or sequence of tensors).

    Mirrors the dtype/alignment asserts of ``kraken/comm/one_shot_all_reduce.py:79-80``.
    """
    return PeerBuffers(stacked)


def stage_input(peers: PeerBuffers, input_tensor: torch.Tensor | None, rank: int, stage: bool = False) -> PeerBuffers:
    """Make ``input_tensor`` the source of rank ``rank`` and return the buffers to reduce.

    The reference kernels first copy the input into this rank's symmetric buffer, where the
    peers read it (``kraken/fused/one_shot_all_reduce_bias.py:56-65``,
    ``one_shot_all_reduce_bias_rms_norm.py:57-61``).  On one GPU nobody else reads that buffer, so
    by default the input is read in place: the returned buffers are the W sources as a pointer
    table whose entry ``rank`` is the input itself -- no copy, no extra launch, the same bits.
    ``stage=True`` keeps the side effect for callers who want the buffer to hold the input
    afterwards: one device copy into the buffer in front of the kernel.  An input that is not
    contiguous or not 16-byte aligned is always copied.
    """
    if input_tensor is None:
        return peers
    n = input_tensor.numel()
    dst = peers.slice(rank).reshape(-1)[:n]
    if dst.data_ptr() == input_tensor.data_ptr():
        return peers
    if stage or not input_tensor.is_contiguous() or input_tensor.data_ptr() % 16 != 0:
        dst.copy_(input_tensor.reshape(-1))
        return peers
    sources = [peers.slice(r).reshape(-1) for r in range(peers.W)]
    sources[rank] = input_tensor.reshape(-1)
    return _Sources(sources, peers.cap)


class _Sources(PeerBuffers):
    """W flat sources of possibly different lengths (each at least as long as the message)."""

    def __init__(self, sources: Sequence[torch.Tensor], cap: int):
        self.W = len(sources)
        self.cap = cap
        self.stride = None
        self.stacked = None
        self.tensors = list(sources)


def bias_args(bias: torch.Tensor | None, numel: int, D: int) -> tuple[int | None, int]:
    """Return (pointer, bias_numel) for a bias of the input's shape or of shape [D]."""
    if bias is None:
        return None, 0
    assert bias.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    assert bias.is_contiguous()
    assert bias.numel() in (numel, D), (
        f"bias must have the shape of the input ({numel} elements) or be a vector of the last dim ({D})"
    )
    return _lib.ptr(bias), bias.numel()
