"""Two-shot all-reduce, this rank's share (``kraken/comm/two_shot_all_reduce.py``)."""
from __future__ import annotations

import torch

from .. import _lib
from ._common import check_stack


def _share_rows(one: torch.Tensor, rank: int, W: int) -> tuple[int, int, tuple[int, ...]]:
    """Contiguous 1/W chunk of a slice ``one``: (offset, numel, shape)."""
    numel = one.numel()
    assert numel % W == 0, "the number of elements must be divisible by the world size"
    share = numel // W
    shape = tuple(one.shape)
    if len(shape) >= 1 and shape[0] % W == 0:
        out_shape = (shape[0] // W, *shape[1:])
    else:
        out_shape = (share,)
    return rank * share, share, out_shape


def two_shot_all_reduce(tensor, **kwargs) -> torch.Tensor:
    """Reduce the 1/W share that rank ``rank`` owns in a two-shot all-reduce.

    Counterpart of ``kraken.comm.two_shot_all_reduce``
    (``kraken/comm/two_shot_all_reduce.py:100-157``).  In the reference every
    rank reduces its share (``:51-62``) and broadcasts it to all peers
    (``:64-67``); with one GPU only the first half exists, so the function
    returns the share.  kwargs:

    * ``rank`` (default 0): which share; ``rank=None`` computes all W shares,
      i.e. the full all-reduced tensor.
    * ``layout``: ``"rows"`` (default) — share = contiguous chunk ``rank`` of
      the flattened slice (``[rows/W, ...]`` when the leading dim divides);
      ``"striped"`` — the reference's ownership: elements
      ``[rank*BLOCK_SIZE, (rank+1)*BLOCK_SIZE)`` of every stripe of
      ``BLOCK_SIZE*W`` elements (``:54,146``), returned compactly as 1-D.
    * ``BLOCK_SIZE`` (default 2048): stripe block for ``layout="striped"``.

    ``tensor`` is the ``[W, ...]`` stack or a list of W separate tensors.
    ``max_num_blocks`` and ``num_warps`` are accepted and ignored.
    """
    peers = check_stack(tensor)
    W, numel = peers.W, peers.cap
    assert numel % 8 == 0, "The number of elements must be 128-bit aligned."
    rank = kwargs.get("rank", 0)
    layout = kwargs.get("layout", "rows")
    block = kwargs.get("BLOCK_SIZE", 2048)
    assert block % W == 0, "BLOCK_SIZE must be divisible by world_size for two-shot all-reduce"
    assert layout in ("rows", "striped")
    dev = _lib.require_device(*peers.tensors)
    lib = _lib.load()
    stream = _lib.current_stream(dev)
    if rank is None:
        out = torch.empty(peers.slice(0).shape, dtype=torch.bfloat16, device=dev)
        rc = peers.reduce(0, numel, None, 0, 0, 0, out.data_ptr(), stream)
        _lib.check(rc, "two_shot_all_reduce")
        return out
    assert 0 <= rank < W
    if layout == "striped":
        share = lib.kr_striped_share_numel(numel, W, block, rank)
        _lib.check(min(share, 0), "two_shot_all_reduce")
        out = torch.empty((share,), dtype=torch.bfloat16, device=dev)
        rc = peers.reduce_striped(numel, None, block, rank, out.data_ptr(), stream)
        _lib.check(rc, "two_shot_all_reduce")
        return out
    off, share, out_shape = _share_rows(peers.slice(0), rank, W)
    assert share % 8 == 0, "each rank's share must be 128-bit aligned"
    out = torch.empty(out_shape, dtype=torch.bfloat16, device=dev)
    rc = peers.reduce(off, share, None, 0, 0, 0, out.data_ptr(), stream)
    _lib.check(rc, "two_shot_all_reduce")
    return out
