"""GEMM + copy-engine reduce-scatter, local arithmetic (``kraken/fused/gemm_reduce_scatter_ce_persistent.py``)."""
from __future__ import annotations

import torch

from .. import _lib
from . import _gemm


def reduce(inp: torch.Tensor, output: torch.Tensor, configs: dict) -> torch.Tensor:
    """Rotated-order W-way band reduce of ``inp [M, N]`` into ``output [M/W, N]``.

    Counterpart of ``reduce`` / ``_reduce_persistent_kernel``
    (``kraken/fused/gemm_reduce_scatter_ce_persistent.py:245-321``):
    ``output = sum_i inp[band (i + RANK + 1) % W]``, accumulated in the input
    dtype (bf16 rounding after every add) unless ``configs["fp32_acc"]``.
    """
    M, N = inp.shape
    W, rank = configs["WORLD_SIZE"], configs["RANK"]
    m_per_rank = M // W
    assert output.shape[0] == m_per_rank and M % W == 0
    assert inp.dtype == torch.bfloat16 and output.dtype == torch.bfloat16
    assert inp.is_contiguous() and output.is_contiguous()
    dev = _lib.require_device(inp, output)
    rc = _lib.load().kr_reduce_rotated_bf16(
        inp.data_ptr(), W, m_per_rank, N, rank, int(not configs.get("fp32_acc", False)),
        output.data_ptr(), _lib.current_stream(dev),
    )
    _lib.check(rc, "gemm_reduce_scatter_ce_persistent.reduce")
    return output


def gemm_reduce_scatter_ce_persistent(
    a: torch.Tensor,
    b: torch.Tensor,
    reduce_op: str = "sum",
    group=None,
    **kwargs,
) -> torch.Tensor:
    """Producer GEMM, band exchange, then the rotated-order band reduce.

    Counterpart of ``kraken.fused.gemm_reduce_scatter_ce_persistent``
    (``kraken/fused/gemm_reduce_scatter_ce_persistent.py:324-375``).  The
    producer GEMM writes the full bf16 ``C = a @ b``; the copy-engine scatter of
    the reference (``:137-175``) is stood in for by assembling the scatter
    buffer ``[W, M/W, N]`` from this rank's own band of C (slot ``rank``) and
    the pre-staged ``peers`` (kwarg, ``[W-1, M/W, N]``, the other ranks in
    ascending order); the reduce then sums the W bands starting at
    ``rank + 1`` (``:258-279``).  kwargs ``rank`` (default 0), ``world_size``.
    """
    assert reduce_op == "sum", "only support sum for now"
    assert a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    a2, b2 = _gemm.prepare_operands(a, b)
    M, N = a2.shape[0], b2.shape[1]
    peers = kwargs.get("peers")
    world_size = kwargs.get("world_size", _gemm.n_peers_of(peers) + 1)
    rank = kwargs.get("rank", 0)
    assert M % world_size == 0
    m_per_rank = M // world_size
    P, _ = _gemm.check_peers(peers, m_per_rank, N)
    assert P == world_size - 1
    gemm_out = torch.empty((M, N), dtype=a.dtype, device=a.device)
    # band_rows = 0: every row of C goes to gemm_out
    _gemm.launch("gemm_reduce_scatter_ce_persistent", a2, b2, M, N, None, 0, 0, None, 0, 0, gemm_out, None, 0)
    scatter_out = torch.empty((world_size, m_per_rank, N), dtype=a.dtype, device=a.device)
    scatter_out[rank].copy_(gemm_out[rank * m_per_rank:(rank + 1) * m_per_rank])
    if P:
        others = [r for r in range(world_size) if r != rank]
        for j, r in enumerate(others):
            scatter_out[r].copy_(peers[j])
    output = torch.empty((m_per_rank, N), dtype=a.dtype, device=a.device)
    configs = {"RANK": rank, "WORLD_SIZE": world_size, "fp32_acc": kwargs.get("fp32_acc", False)}
    return reduce(scatter_out.view(M, N), output, configs)
