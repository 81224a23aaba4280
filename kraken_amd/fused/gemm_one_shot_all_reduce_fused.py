"""GEMM + one-shot all-reduce, local arithmetic (``kraken/fused/gemm_one_shot_all_reduce_fused.py``)."""
from __future__ import annotations

import torch

from . import _gemm


def gemm_one_shot_all_reduce(a: torch.Tensor, b: torch.Tensor, **kwargs) -> torch.Tensor:
    """``out = a @ b + sum_j peers[j] (+ bias)`` with the sum fused into the GEMM epilogue.

    Counterpart of ``kraken.fused.gemm_one_shot_all_reduce_fused``
    (``kraken/fused/gemm_one_shot_all_reduce_fused.py:106-178``; arithmetic
    ``:56-99``).  In the reference every rank stores its fp32 partial product to
    symmetric memory and re-reads all W of them; here the W-1 partials of the
    other ranks arrive pre-staged and this rank's partial never leaves the
    accumulators.  kwargs:

    * ``peers``: bf16 ``[W-1, M, N]`` partial products of the other ranks (or a
      list of W-1 separate ``[M, N]`` tensors), or ``None`` (W = 1: plain GEMM);
    * ``bias``: bf16 ``[N]`` or ``None`` (the reference has no bias here);
    * ``out_dtype``: ``torch.float32`` (default — the reference's output
      dtype, ``:135``) or ``torch.bfloat16``.

    ``group``, ``BLOCK_SIZE_M/N/K``, ``GROUP_SIZE_M``, ``num_warps`` and
    ``num_stages`` are accepted and ignored.
    """
    a, b = _gemm.prepare_operands(a, b)
    M, N = a.shape[0], b.shape[1]
    assert N % 8 == 0, "N must be a multiple of 8"
    peers = kwargs.get("peers")
    bias = kwargs.get("bias")
    out_dtype = kwargs.get("out_dtype", torch.float32)
    assert out_dtype in (torch.float32, torch.bfloat16)
    P, pstride = _gemm.check_peers(peers, M, N)
    if bias is not None:
        assert bias.dtype == torch.bfloat16 and bias.shape == (N,) and bias.is_contiguous()
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    _gemm.launch("gemm_one_shot_all_reduce", a, b, M, N, peers, P, pstride, bias, 0, M, None, out, 0)
    return out
