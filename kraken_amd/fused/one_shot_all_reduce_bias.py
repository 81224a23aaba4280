"""One-shot all-reduce + bias, local arithmetic (``kraken/fused/one_shot_all_reduce_bias.py``)."""
from __future__ import annotations

import torch

from .. import _lib
from ..comm._common import bias_args, check_stack, stage_input


def one_shot_all_reduce_bias(
    symm_mem_buffer,
    input_tensor: torch.Tensor | None,
    bias: torch.Tensor | None,
    output: torch.Tensor,
    max_num_blocks: int = 24,
    BLOCK_SIZE: int = 4096,
    group=None,
    *,
    rank: int = 0,
    stage: bool = False,
) -> None:
    """``output = bias + sum over the W slices`` (bias first, then slices 0..W-1, fp32).

    Counterpart of ``kraken.fused.one_shot_all_reduce_bias``
    (``kraken/fused/one_shot_all_reduce_bias.py:105-173``; arithmetic ``:76-94``).

    ``symm_mem_buffer`` is the ``[W, ...]`` stack standing in for the peers'
    symmetric-memory buffers, or a list of W separate tensors; each slice may be larger than the input, only its
    first ``output.numel()`` elements are used (the reference rendezvouses on a
    buffer larger than the message as well, ``test/test_allreduce_bias.py:57-62``).
    ``input_tensor``, if given, is rank ``rank``'s contribution in place of slice ``rank``:
    it is read where it lies, inside the one kernel (the reference's fused copy-in ``:56-65``
    exists so that the peers can read it; here nobody else does); ``stage=True`` also copies it
    into slice ``rank`` first, for callers who want that side effect.  Pass ``None`` when the
    stack is already staged.  ``bias`` has the shape of the input (as the reference passes it)
    or is a vector over the last dimension, or ``None`` (plain sum, ``:80-84``).
    ``max_num_blocks``, ``BLOCK_SIZE`` and ``group`` are accepted and ignored.
    """
    if symm_mem_buffer is None:
        raise ValueError("symm_mem_buffer much be a valid symmetric memory tensor.")
    peers = check_stack(symm_mem_buffer)
    W, cap = peers.W, peers.cap
    ref = input_tensor if input_tensor is not None else output
    assert ref.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    numel = ref.numel()
    assert numel % 8 == 0, "The number of elements must be 128-bit aligned."
    assert output.dtype == torch.bfloat16 and output.numel() == numel and output.is_contiguous()
    assert numel <= cap, "the message does not fit in one slice of the stacked buffer"
    assert 0 <= rank < W
    D = ref.shape[-1] if ref.dim() >= 1 else numel
    bias_ptr, bias_numel = bias_args(bias, numel, D)
    dev = _lib.require_device(*peers.tensors, input_tensor, bias, output)
    peers = stage_input(peers, input_tensor, rank, stage)
    rc = peers.reduce(0, numel, bias_ptr, bias_numel, D, 1, output.data_ptr(), _lib.current_stream(dev))
    _lib.check(rc, "one_shot_all_reduce_bias")
