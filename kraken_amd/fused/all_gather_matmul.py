"""All-gather + matmul, local arithmetic (``kraken/fused/all_gather_matmul.py``)."""
from __future__ import annotations

import torch

from . import _gemm


def all_gather_matmul(
    a_shared: torch.Tensor,
    b: torch.Tensor,
    a_out: torch.Tensor | None = None,
    progress: torch.Tensor | None = None,
    **kwargs,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``c = concat_r(a_shared[r]) @ b``; returns ``(a_gathered, c)``.

    Counterpart of ``kraken.fused.all_gather_matmul``
    (``kraken/fused/all_gather_matmul.py:222-325``; arithmetic ``:87-123``).
    ``a_shared`` is the ``[W, m, K]`` stack of all ranks' shards — already
    "gathered" on one GPU — so ``a_gathered`` is its zero-copy ``[W*m, K]``
    view (copied into ``a_out`` when one is passed).  ``b`` must satisfy
    ``b.T.is_contiguous()`` like in the reference (``:158-160``).  The order of
    the M tiles is rotated so that the shard of ``rank`` (kwarg, default 0) is
    consumed first (``:93``); this changes scheduling only.  ``progress``, if
    given, is set to 1 everywhere (all chunks present).  Tile-size kwargs
    (``splits_per_rank``, ``block_size_*``, ``group_size_m``, ``num_stages``,
    ``num_warps``) are accepted and ignored.
    """
    assert a_shared.dim() == 3, "expected the stacked shards [W, m, K]"
    assert a_shared.dtype == torch.bfloat16 and b.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    assert a_shared.is_contiguous()
    W, m, K = a_shared.shape
    assert b.dim() == 2 and b.shape[0] == K
    if not b.T.is_contiguous():
        raise ValueError("b.T must be contiguous")
    rank = kwargs.get("rank", 0)
    assert 0 <= rank < W
    a_full = a_shared.reshape(W * m, K)
    if a_out is not None:
        assert a_out.shape == a_full.shape and a_out.dtype == a_full.dtype
        a_out.copy_(a_full)
    else:
        a_out = a_full
    if progress is not None:
        progress.fill_(1)
    a2, b2 = _gemm.prepare_operands(a_full, b)
    M, N = W * m, b.shape[1]
    assert N % 8 == 0, "N must be a multiple of 8"
    c = torch.empty((M, N), dtype=a_shared.dtype, device=a_shared.device)
    _gemm.launch("all_gather_matmul", a2, b2, M, N, None, 0, 0, None, 0, M, None, c, rank * m)
    return a_out, c
