"""One-shot all-reduce, local arithmetic (``kraken/comm/one_shot_all_reduce.py``)."""
from __future__ import annotations

import torch

from .. import _lib
from ._common import check_stack


def one_shot_all_reduce(tensor, **kwargs) -> torch.Tensor:
    """``output = sum over the W slices of tensor`` (one kernel, every element).

    Counterpart of ``kraken.comm.one_shot_all_reduce``
    (``kraken/comm/one_shot_all_reduce.py:57-113``).  ``tensor`` is the
    ``[W, ...]`` stack standing in for the W peers' symmetric-memory buffers,
    or a list of W separately allocated tensors (a pointer table is then
    passed to the kernel, as ``buffer_ptrs_dev`` is in the reference, ``:96``);
    the result has the shape of one slice.  The sum is accumulated in fp32 in
    ascending slice order and rounded to bf16 once (the reference kernel
    accumulates in bf16, ``:40-46``; its test tolerance of 1e-1 covers both).

    ``max_num_blocks``, ``num_warps`` and ``BLOCK_SIZE`` are accepted for
    signature compatibility and ignored: the launch is sized to fill the GPU.
    """
    peers = check_stack(tensor)
    numel = peers.cap
    assert numel % 8 == 0, "The number of elements must be 128-bit aligned."
    dev = _lib.require_device(*peers.tensors)
    out = torch.empty(peers.slice(0).shape, dtype=torch.bfloat16, device=dev)
    rc = peers.reduce(0, numel, None, 0, 0, 1, out.data_ptr(), _lib.current_stream(dev))
    _lib.check(rc, "one_shot_all_reduce")
    return out
