"""One-shot all-reduce + bias + RMSNorm (``kraken/fused/one_shot_all_reduce_bias_rms_norm.py``)."""
from __future__ import annotations

import math

import torch

from .. import _lib
from ..comm._common import check_stack, stage_input


def _launch_reduce_rms_norm(name, symm_mem_input, x, bias, w, y, eps, rank, stage=False):
    D = y.shape[-1]
    if x is not None:
        assert y.shape == x.shape
        assert y.dtype == x.dtype
        assert y.stride() == x.stride(), (str(x.stride()), str(y.stride()))
        assert x.is_contiguous()
    assert w.is_contiguous()
    assert w.shape == (D,)
    assert y.is_contiguous()
    assert y.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    assert D % 8 == 0, "The row length must be 128-bit aligned."
    peers = check_stack(symm_mem_input)
    W, cap = peers.W, peers.cap
    rows = math.prod(y.shape[:-1])
    assert rows * D <= cap, "the message does not fit in one slice of the stacked buffer"
    assert 0 <= rank < W
    bias_is_vector = 0
    if bias is not None:
        assert bias.dtype == torch.bfloat16 and bias.is_contiguous()
        assert bias.numel() in (rows * D, D), "bias must have the shape of x or be a vector of the last dim"
        bias_is_vector = int(bias.numel() == D and rows != 1)
    dev = _lib.require_device(*peers.tensors, x, bias, w, y)
    peers = stage_input(peers, x, rank, stage)
    rc = peers.reduce_rmsnorm(rows, D, _lib.ptr(bias), bias_is_vector, w.data_ptr(), float(eps), y.data_ptr(),
                              _lib.current_stream(dev))
    _lib.check(rc, name)


def one_shot_all_reduce_bias_rms_norm(
    symm_mem_input,
    x: torch.Tensor | None,
    bias: torch.Tensor | None,
    w: torch.Tensor,
    y: torch.Tensor,
    eps: float = 1.0e-5,
    BLOCK_SIZE: int = 1024,
    group=None,
    *,
    rank: int = 0,
    stage: bool = False,
) -> None:
    """``y = rms_norm(bias + sum over the W slices, w, eps)``, one pass over the input.

    Counterpart of ``kraken.fused.one_shot_all_reduce_bias_rms_norm``
    (``kraken/fused/one_shot_all_reduce_bias_rms_norm.py:102-169``; arithmetic
    ``:73-91``): per row, ``s = fp32(bias) + x_0 + ... + x_{W-1}`` in fp32,
    ``y = bf16(s * rsqrt(mean(s^2) + eps) * fp32(w))``.

    ``symm_mem_input`` is the ``[W, ...]`` stack or a list of W separate
    tensors; ``x``, if given, is read in place as rank ``rank``'s
    contribution (the reference's copy-in ``:57-61`` serves the peers, of which there are none
    here; ``stage=True`` also copies it into slice ``rank`` first); pass ``None`` when the stack
    is already staged.  ``bias`` has the shape of
    ``x`` (reference usage) or ``[D]``.  ``BLOCK_SIZE``/``group`` are ignored.
    """
    _launch_reduce_rms_norm("one_shot_all_reduce_bias_rms_norm", symm_mem_input, x, bias, w, y, eps, rank, stage)
