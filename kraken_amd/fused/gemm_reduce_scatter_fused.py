"""GEMM + reduce-scatter, local arithmetic (``kraken/fused/gemm_reduce_scatter_fused.py``)."""
from __future__ import annotations

import torch

from . import _gemm


def gemm_reduce_scatter(a: torch.Tensor, b: torch.Tensor, **kwargs) -> torch.Tensor:
    """``out = (a @ b)[band] + sum_j peers[j]`` for this rank's ``M/W``-row band.

    Counterpart of ``kraken.fused.gemm_reduce_scatter``
    (``kraken/fused/gemm_reduce_scatter_fused.py:152-235``; arithmetic
    ``:63-72,102-145``).  Like the reference, the full ``M x N`` product is
    computed (the other ranks need the other bands): rows outside the band are
    written as bf16 to ``c_scratch`` (the stand-in for this rank's symmetric
    buffer), rows inside it are summed with the W-1 pre-staged partials in
    the epilogue and written once to the ``[M/W, N]`` result.  The own partial
    stays in fp32 (the reference rounds it to the input dtype first, ``:72``).
    kwargs:

    * ``peers``: bf16 ``[W-1, M/W, N]`` (or a list of W-1 separate ``[M/W, N]``
      tensors) — the other ranks' partials of this rank's band; ``None`` means W = ``world_size`` (default 1) without peers;
    * ``rank`` (default 0), ``world_size`` (default ``len(peers)+1``);
    * ``c_scratch``: bf16 ``[M, N]`` buffer for the other bands; allocated if
      ``None``; pass ``False`` to skip writing them.

    Returns ``[M/W, N]`` in ``a.dtype``.  Tile-size kwargs are ignored.
    """
    in_dtype = a.dtype
    a, b = _gemm.prepare_operands(a, b)
    M, N = a.shape[0], b.shape[1]
    assert N % 8 == 0, "N must be a multiple of 8"
    peers = kwargs.get("peers")
    world_size = kwargs.get("world_size", _gemm.n_peers_of(peers) + 1)
    rank = kwargs.get("rank", 0)
    assert M % world_size == 0, f"M dimension ({M}) must be divisible by world_size ({world_size})"
    assert 0 <= rank < world_size
    m_scatter = M // world_size
    P, pstride = _gemm.check_peers(peers, m_scatter, N)
    assert P in (0, world_size - 1), "peers must hold the partials of the other world_size-1 ranks"
    c_scratch = kwargs.get("c_scratch")
    if c_scratch is None:
        c_scratch = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    elif c_scratch is False:
        c_scratch = None
    else:
        assert c_scratch.dtype == torch.bfloat16 and tuple(c_scratch.shape) == (M, N) and c_scratch.is_contiguous()
    out = torch.empty((m_scatter, N), dtype=in_dtype, device=a.device)
    # tile order rotated so that the band's tiles (the ones with extra epilogue traffic) run first
    _gemm.launch("gemm_reduce_scatter", a, b, M, N, peers, P, pstride, None,
                 rank * m_scatter, m_scatter, c_scratch, out, rank * m_scatter)
    return out
