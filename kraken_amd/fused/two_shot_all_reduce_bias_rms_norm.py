"""Two-shot all-reduce + bias + RMSNorm (``kraken/fused/two_shot_all_reduce_bias_rms_norm.py``)."""
from __future__ import annotations

import math

import torch

from ..comm._common import check_stack
from .one_shot_all_reduce_bias_rms_norm import _launch_reduce_rms_norm


def two_shot_all_reduce_bias_rms_norm(
    symm_mem_input,
    x: torch.Tensor | None,
    bias: torch.Tensor | None,
    w: torch.Tensor,
    y: torch.Tensor,
    eps: float = 1.0e-5,
    group=None,
    *,
    rank: int = 0,
    stage: bool = False,
) -> None:
    """Same result as the one-shot variant; keeps the two-shot variant's shape rules.

    Counterpart of ``kraken.fused.two_shot_all_reduce_bias_rms_norm``
    (``kraken/fused/two_shot_all_reduce_bias_rms_norm.py:132-223``).  The
    reference splits each block of ``rows_per_block`` rows into W slices of
    ``size_per_rank`` elements and asserts the split is exact and a multiple
    of 16 (``:176-199``); those asserts are kept so that callers fail in the
    same places.  On one GPU there is no broadcast step, so the reduced row
    stays in fp32 registers up to the norm (the reference rounds it to bf16
    in its symmetric buffer in between, ``:96-99,110-121``; the difference is
    below one bf16 ulp of the row values).
    """
    D = y.shape[-1]
    total_rows = math.prod(y.shape[:-1])
    if total_rows < 2:
        rows_per_block = 1
    elif total_rows <= 32:
        rows_per_block = 2
    elif total_rows <= 64:
        rows_per_block = 4
    else:
        rows_per_block = 8
    W = check_stack(symm_mem_input).W
    size_per_rank = rows_per_block * D // W
    assert size_per_rank * W == rows_per_block * D
    assert size_per_rank % 16 == 0
    _launch_reduce_rms_norm("two_shot_all_reduce_bias_rms_norm", symm_mem_input, x, bias, w, y, eps, rank, stage)
