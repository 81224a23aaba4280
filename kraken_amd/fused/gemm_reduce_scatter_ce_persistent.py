"""GEMM + copy-engine reduce-scatter, local arithmetic (``kraken/fused/gemm_reduce_scatter_ce_persistent.py``)."""
from __future__ import annotations

import torch

from .. import _lib, _waits
from ..comm.copy_engine_all_gather import _get_backend_stream
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


def gemm_producer_w_progress(
    a: torch.Tensor,
    b: torch.Tensor,
    gemm_out: torch.Tensor,
    progress: torch.Tensor,
    signal_pad: torch.Tensor,
    configs: dict,
    group=None,
) -> None:
    """``gemm_out = a @ b`` with one completion flag per destination rank's band.

    Counterpart of ``gemm_producer_w_progress`` / ``_gemm_producer_persistent_kernel``
    (``kraken/fused/gemm_reduce_scatter_ce_persistent.py:46-134,178-242``): the M
    tiles are processed starting at the band of ``RANK + 1`` (``:88,102``); every
    finished tile is counted into ``progress[r]`` of the bands it touches and the
    tile that completes band ``r`` sets ``signal_pad[r] = 1`` (``:117-132``).  Both
    are 32-bit integer tensors of ``WORLD_SIZE`` elements, zeroed by the caller
    (``:364-365``).  Shapes whose output tiles all run at once (one round of the
    compute units or less) finish all bands together, so for those the library's
    fastest GEMM is used when it is a split one (K loop shared between workgroups):
    their flags are set by a stream-ordered fill behind the GEMM and ``progress``
    is not counted.  Every larger shape runs the producer kernel, whose bands
    finish, and are flagged, one after the other.
    """
    a2, b2 = _gemm.prepare_operands(a, b)
    M, N = a2.shape[0], b2.shape[1]
    W, rank = configs["WORLD_SIZE"], configs["RANK"]
    assert M % W == 0 and 0 <= rank < W
    assert gemm_out.shape == (M, N) and gemm_out.dtype == torch.bfloat16 and gemm_out.is_contiguous()
    for t in (progress, signal_pad):
        assert t.dtype in (torch.int32, torch.uint32) and t.is_contiguous() and t.numel() >= W
    dev = _lib.require_device(a2, b2, gemm_out, progress, signal_pad)
    lib = _lib.load()
    pivot = ((rank + 1) % W) * (M // W)
    one_round = -(-M // 256) * -(-N // 256) <= torch.cuda.get_device_properties(dev).multi_processor_count
    if one_round and lib.kr_gemm_workspace_bytes(M, N, a2.shape[1]) > 0:
        _gemm.launch("gemm_producer_w_progress", a2, b2, M, N, None, 0, 0, None, 0, 0, gemm_out, None, pivot)
        signal_pad.fill_(1)
        return
    rc = lib.kr_gemm_producer_bf16(
        a2.data_ptr(), a2.stride(0), a2.stride(1), b2.data_ptr(), b2.stride(0), b2.stride(1),
        M, N, a2.shape[1], gemm_out.data_ptr(), W, rank, progress.data_ptr(), signal_pad.data_ptr(),
        _lib.current_stream(dev),
    )
    _lib.check(rc, "gemm_producer_w_progress")


def copy_engine_scatter(
    inp: torch.Tensor,
    output,
    signal_pad: torch.Tensor,
    group=None,
    *,
    rank: int = 0,
    wait_limit_us: int = 0,
    status: torch.Tensor | None = None,
    copy_engine: bool = False,
) -> None:
    """Copy every finished band of ``inp [M, N]`` to its destination, on the current stream.

    Counterpart of ``copy_engine_scatter``
    (``kraken/fused/gemm_reduce_scatter_ce_persistent.py:137-175``): for
    ``step = 0..W-1`` the band of ``remote = (rank + step + 1) % W`` is copied once
    ``signal_pad[remote] == 1`` — a stream-ordered wait in front of each copy
    (``:153-163``), so the copies start while the producer GEMM is still running on
    another stream.  ``output`` holds the W destinations: a ``[W, M/W, N]`` tensor or
    a sequence of W tensors ``[M/W, N]`` (``None`` entries are skipped: no wait, no
    copy); ``output[r]`` stands for slot ``rank`` of rank r's symmetric buffer
    (``:165-169``).  The waits are bounded (``wait_limit_us``, default 5 s); a wait
    that runs out sets ``status`` (int32 ``[1]``, zeroed by the caller) to 1 and the bands copied
    behind it are invalid; without ``status`` the wrapper keeps a word of its own and the next call
    of an overlap function (or ``kraken_amd._waits.check()``) raises once the copies have run.  The
    copies are ordinary copy kernels; ``copy_engine=True`` hands them to the GPU's
    copy engines (``kr_copy_engine_memcpy``).
    """
    M, N = inp.shape
    W = len(output)
    assert M % W == 0 and 0 <= rank < W
    m_per_rank = M // W
    assert signal_pad.dtype in (torch.int32, torch.uint32) and signal_pad.is_contiguous() and signal_pad.numel() >= W
    dev = _lib.require_device(inp, signal_pad, status, *[t for t in output if t is not None])
    lib = _lib.load()
    stream = _lib.current_stream(dev)
    _waits.check()
    own_status = status is None
    if own_status:
        status = _waits.new_status(dev)     # shared by the W waits: after one runs out the others give up at once
    for step in range(W):
        remote = (rank + step + 1) % W
        dst = output[remote]
        if dst is None:
            continue
        assert tuple(dst.shape) == (m_per_rank, N) and dst.dtype == inp.dtype
        rc = lib.kr_stream_wait_value32(signal_pad.data_ptr() + 4 * remote, 1, wait_limit_us, _lib.ptr(status), stream)
        _lib.check(rc, "stream_wait_value32")
        band = inp[remote * m_per_rank:(remote + 1) * m_per_rank]
        if copy_engine and dst.is_contiguous() and band.is_contiguous():
            _lib.copy_engine_copy(dst, band, stream)
        else:
            dst.copy_(band)
    if own_status:
        _waits.watch(status, "copy_engine_scatter")


def gemm_reduce_scatter_ce_persistent(
    a: torch.Tensor,
    b: torch.Tensor,
    reduce_op: str = "sum",
    group=None,
    **kwargs,
) -> torch.Tensor:
    """Producer GEMM, band exchange on a side stream, then the rotated-order band reduce.

    Counterpart of ``kraken.fused.gemm_reduce_scatter_ce_persistent``
    (``kraken/fused/gemm_reduce_scatter_ce_persistent.py:324-375``).  The producer
    GEMM writes the full bf16 ``C = a @ b`` on the current stream and flags every
    band as it completes; a side stream, which first waits for the current stream
    (``:345-346``), copies each flagged band to its destination (``:367-368``).  On
    one GPU the destinations are: this rank's own band -> slot ``rank`` of the
    scatter buffer ``[W, M/W, N]``; the bands of the other ranks -> ``sent[r]`` when
    the kwarg ``sent`` (``[W, M/W, N]`` tensor or sequence) is given, else nowhere
    (the own band, the last to finish, is then copied in stream order behind the
    GEMM and no flag is waited for).
    What the other ranks would push arrives from the pre-staged ``peers`` (kwarg,
    ``[W-1, M/W, N]``, the other ranks in ascending order), copied on the side
    stream while the GEMM runs.  The current stream then waits for the side stream
    (``:370``) and the reduce sums the W bands starting at ``rank + 1``
    (``:258-279``).  kwargs ``rank`` (default 0), ``world_size``, ``fp32_acc``,
    ``wait_limit_us``, ``status``, ``copy_engine``.
    """
    assert reduce_op == "sum", "only support sum for now"
    assert a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    M, N = a.shape[0], b.shape[1]
    peers = kwargs.get("peers")
    world_size = kwargs.get("world_size", _gemm.n_peers_of(peers) + 1)
    rank = kwargs.get("rank", 0)
    assert M % world_size == 0
    m_per_rank = M // world_size
    P, _ = _gemm.check_peers(peers, m_per_rank, N)
    assert P == world_size - 1
    dev = _lib.require_device(a, b)
    _waits.check()      # an earlier call's failed wait is reported before anything of this call is enqueued
    gemm_out = torch.empty((M, N), dtype=a.dtype, device=dev)
    scatter_out = torch.empty((world_size, m_per_rank, N), dtype=a.dtype, device=dev)
    output = torch.empty((m_per_rank, N), dtype=a.dtype, device=dev)
    configs = {"RANK": rank, "WORLD_SIZE": world_size, "fp32_acc": kwargs.get("fp32_acc", False)}
    if M == 0 or N == 0:
        return output
    progress = torch.zeros(world_size, dtype=torch.int32, device=dev)
    signal_pad = torch.zeros(world_size, dtype=torch.int32, device=dev)
    sent = kwargs.get("sent")
    dests = [None if sent is None else sent[r] for r in range(world_size)]
    dests[rank] = scatter_out[rank]

    current = torch.cuda.current_stream(dev)
    backend_stream = _get_backend_stream(dev)
    backend_stream.wait_stream(current)
    gemm_producer_w_progress(a, b, gemm_out, progress, signal_pad, configs)
    with torch.cuda.stream(backend_stream):
        if isinstance(peers, torch.Tensor):
            # the other ranks in ascending order: two runs, below and above the own slot
            scatter_out[:rank].copy_(peers[:rank])
            scatter_out[rank + 1:].copy_(peers[rank:])
        else:
            others = [r for r in range(world_size) if r != rank]
            for j, r in enumerate(others):
                scatter_out[r].copy_(peers[j])
        if sent is not None:
            copy_engine_scatter(gemm_out, dests, signal_pad, rank=rank,
                                wait_limit_us=kwargs.get("wait_limit_us", 0), status=kwargs.get("status"),
                                copy_engine=kwargs.get("copy_engine", False))
    if sent is None:
        # only the own band has a destination on this GPU, and it is the last one the GEMM
        # finishes: its copy gains nothing from a flag and goes behind the GEMM in stream order
        scatter_out[rank].copy_(gemm_out[rank * m_per_rank:(rank + 1) * m_per_rank])
    current.wait_stream(backend_stream)
    return reduce(scatter_out.view(M, N), output, configs)
