"""One-shot all-reduce, local arithmetic (``kraken/comm/one_shot_all_reduce.py``)."""
from __future__ import annotations

import torch

from .. import _lib
from ._common import check_stack


def one_shot_all_reduce(tensor: torch.Tensor, **kwargs) -> torch.Tensor:
    """``output = sum over the W slices of tensor`` (one kernel, every element).

    Counterpart of ``kraken.comm.one_shot_all_reduce``
    (``kraken/comm/one_shot_all_reduce.py:57-113``).  ``tensor`` is the
    ``[W, ...]`` stack standing in for the W peers' symmetric-memory buffers;
    the result has the shape of one slice.  The sum is accumulated in fp32 in
    ascending slice order and rounded to bf16 once (the reference kernel
    accumulates in bf16, ``:40-46``; its test tolerance of 1e-1 covers both).

    ``max_num_blocks``, ``num_warps`` and ``BLOCK_SIZE`` are accepted for
    signature compatibility and ignored: the launch is sized to fill the GPU.
    """
    W, numel, stride = check_stack(tensor)
    assert numel % 8 == 0, "The number of elements must be 128-bit aligned."
    dev = _lib.require_device(tensor)
    out = torch.empty(tensor.shape[1:], dtype=tensor.dtype, device=dev)
    rc = _lib.load().kr_reduce_bf16(
        tensor.data_ptr(), W, stride, numel, None, 0, 0, 1, out.data_ptr(), _lib.current_stream(dev)
    )
    _lib.check(rc, "one_shot_all_reduce")
    return out
