"""All-gather + matmul, local arithmetic (``kraken/fused/all_gather_matmul.py``)."""
from __future__ import annotations

import torch

from .. import _lib, _waits
from ..comm._common import PeerBuffers
from ..comm.copy_engine_all_gather import _copy_engine_all_gather_w_progress
from . import _gemm


def _matmul_w_progress(a, a_local, b, progress, configs, status=None) -> torch.Tensor:
    """``c = a @ b`` where the rows of ``a`` arrive while the kernel runs.

    Counterpart of ``_matmul_w_progress`` (``kraken/fused/all_gather_matmul.py:147-219``):
    tiles of the local shard read ``a_local``, all others wait for
    ``progress[chunk] == 1`` (``:95-110``).  ``configs``: ``RANK``, ``WORLD_SIZE``,
    ``SPLITS_PER_RANK``, optional ``wait_limit_us``.
    """
    M, K = a.shape
    assert b.shape[0] == K
    if not b.T.is_contiguous():
        raise ValueError("b.T must be contiguous")
    N = b.shape[1]
    assert K % 8 == 0 and N % 8 == 0, "K and N must be multiples of 8"
    assert a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    assert a.stride(1) == 1 and (a_local is None or a_local.stride(1) == 1)
    dev = _lib.require_device(a, a_local, b, progress, status)
    c = torch.empty((M, N), device=dev, dtype=a.dtype)
    rc = _lib.load().kr_all_gather_matmul_bf16(
        a.data_ptr(), a.stride(0), _lib.ptr(a_local), 0 if a_local is None else a_local.stride(0),
        b.data_ptr(), b.stride(0), b.stride(1), M, N, K,
        configs["WORLD_SIZE"], configs["RANK"], configs["SPLITS_PER_RANK"],
        _lib.ptr(progress), int(configs.get("wait_limit_us", 0)), _lib.ptr(status),
        c.data_ptr(), _lib.current_stream(dev),
    )
    _lib.check(rc, "all_gather_matmul")
    return c


def _all_gather_matmul_fp8(a_shared, peers: PeerBuffers, b, a_out, progress, **kwargs):
    """The fp8 branch of ``all_gather_matmul`` (``all_gather_matmul.py:53,121,213``): fp8 product with fp32
    accumulation, rounded to fp8 once.  Shapes the fp8 kernel takes (M, N multiples of 256, K of 128) run on
    the fp8 matrix-core instruction (``kr_gemm_fp8``, or ``kr_all_gather_matmul_fp8`` for ``gather=True``: the
    shards are copied chunk by chunk on a side stream while the tiles wait for their chunk's flag, as in the
    bf16 form); others are widened to bf16 (exact), multiplied by the bf16 kernels with an fp32 result, and
    rounded by ``kr_cast_f32_to_fp8`` -- the same sums up to fp32 summation order -- after the gather has
    finished.  ``fp8_kernel=False`` forces the widening path."""
    fp8 = torch.float8_e4m3fn
    W = peers.W
    m, K = peers.slice(0).shape
    assert b.dtype == fp8, "fp8 shards need an fp8 b"
    assert b.dim() == 2 and b.shape[0] == K
    if not b.T.is_contiguous():
        raise ValueError("b.T must be contiguous")
    stacked = peers.stacked is not None and peers.stacked.is_contiguous()
    gather = kwargs.get("gather", not stacked)
    M, N = W * m, b.shape[1]
    assert K % 16 == 0 and N % 16 == 0 and (M * N) % 16 == 0, "fp8 operands: sizes must be multiples of 16"
    rank = kwargs.get("rank", 0)
    assert 0 <= rank < W
    splits = kwargs.get("splits_per_rank", 1)
    dev = _lib.require_device(*peers.tensors, b, a_out, progress)
    lib = _lib.load()
    stream = _lib.current_stream(dev)
    native = kwargs.get("fp8_kernel", True) and M % 256 == 0 and N % 256 == 0 and K % 128 == 0
    if gather:
        assert m % splits == 0, "splits_per_rank must divide the rows of a shard"
        _waits.check()      # an earlier call's failed wait is reported before anything of this call is enqueued
        if a_out is None:
            a_out = torch.empty((M, K), dtype=fp8, device=dev)
        else:
            assert tuple(a_out.shape) == (M, K) and a_out.dtype == fp8 and a_out.is_contiguous()
        if progress is None:
            progress = torch.zeros(W * splits, dtype=torch.int32, device=dev)
        else:
            progress.fill_(0)
        backend_stream = _copy_engine_all_gather_w_progress(a_out, a_shared, progress, splits, rank=rank,
                                                            copy_engine=kwargs.get("copy_engine", False))
        if native:
            status = kwargs.get("status")
            own_status = status is None
            if own_status:
                status = _waits.new_status(dev)
            a_local = peers.slice(rank)
            assert a_local.stride(1) == 1
            c = torch.empty((M, N), dtype=fp8, device=dev)
            rc = lib.kr_all_gather_matmul_fp8(
                a_out.data_ptr(), K, a_local.data_ptr(), a_local.stride(0), b.T.data_ptr(), K, M, N, K, W, rank, splits,
                progress.data_ptr(), int(kwargs.get("wait_limit_us", 0)), _lib.ptr(status), c.data_ptr(), 2, stream)
            _lib.check(rc, "all_gather_matmul(fp8)")
            torch.cuda.current_stream(dev).wait_stream(backend_stream)
            if own_status:
                _waits.watch(status, "all_gather_matmul")
            return a_out, c
        torch.cuda.current_stream(dev).wait_stream(backend_stream)   # no overlap on the widening path
        a_full = a_out
    else:
        assert stacked, "gather=False needs the shards as one contiguous [W, m, K] tensor"
        a_full = peers.stacked.reshape(M, K)
        if a_out is not None:
            assert a_out.shape == a_full.shape and a_out.dtype == fp8
            a_out.copy_(a_full)
        else:
            a_out = a_full
        if progress is not None:
            progress.fill_(1)
    if native:
        c = torch.empty((M, N), dtype=fp8, device=dev)
        _lib.check(lib.kr_gemm_fp8(a_full.data_ptr(), K, b.T.data_ptr(), K, M, N, K, c.data_ptr(), 2, stream),
                   "all_gather_matmul(fp8)")
        return a_out, c
    a16 = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
    bt16 = torch.empty((N, K), dtype=torch.bfloat16, device=dev)           # b.T is contiguous: memory [N, K]
    _lib.check(lib.kr_cast_fp8_to_bf16(a_full.data_ptr(), M * K, a16.data_ptr(), stream), "cast_fp8_to_bf16(a)")
    _lib.check(lib.kr_cast_fp8_to_bf16(b.T.data_ptr(), N * K, bt16.data_ptr(), stream), "cast_fp8_to_bf16(b)")
    c32 = torch.empty((M, N), dtype=torch.float32, device=dev)
    _gemm.launch("all_gather_matmul", a16, bt16.T, M, N, None, 0, 0, None, 0, M, None, c32, rank * m)
    c = torch.empty((M, N), dtype=fp8, device=dev)
    _lib.check(lib.kr_cast_f32_to_fp8(c32.data_ptr(), M * N, c.data_ptr(), stream), "cast_f32_to_fp8(c)")
    return a_out, c


def all_gather_matmul(
    a_shared,
    b: torch.Tensor,
    a_out: torch.Tensor | None = None,
    progress: torch.Tensor | None = None,
    **kwargs,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``c = concat_r(a_shared[r]) @ b``; returns ``(a_gathered, c)``.

    Counterpart of ``kraken.fused.all_gather_matmul``
    (``kraken/fused/all_gather_matmul.py:222-325``; arithmetic ``:87-123``).
    ``a_shared`` holds all ranks' shards: the ``[W, m, K]`` stack or a list of
    W separate ``[m, K]`` tensors.  ``b`` must satisfy ``b.T.is_contiguous()``
    like in the reference (``:158-160``).  Two modes (kwarg ``gather``):

    * ``gather=False`` (default for a contiguous stack): the stack already is
      the gathered matrix, so ``a_gathered`` is its zero-copy ``[W*m, K]`` view
      (copied into ``a_out`` when one is passed), ``progress`` is set to 1
      everywhere and the GEMM waits for nothing.
    * ``gather=True`` (default for a list of shards): the reference's overlap.
      The shards are copied chunk by chunk into ``a_out`` on a side stream,
      each chunk followed by its flag in ``progress`` (``:308-311``), while the
      GEMM on the current stream consumes them: tiles of the local shard
      (``rank``) read it in place, every other tile waits for its chunk's flag
      (``:95-110``).  The current stream then waits for the side stream
      (``:316``).  ``status`` (int32 ``[1]``, zeroed by the caller) receives a
      non-zero value if a tile's wait ran out (``wait_limit_us``, default 5 s) and
      ``c`` is then invalid; without ``status`` the wrapper keeps a word of its own
      and the next call of an overlap function (or ``kraken_amd._waits.check()``)
      raises once the failed call has finished.
      The copies are ordinary copy kernels, which share the compute units with
      the GEMM; ``copy_engine=True`` hands them to the GPU's copy engines.

    In both modes the order of the M tiles is rotated so that the shard of
    ``rank`` (kwarg, default 0) is consumed first and the others in the order
    the copies are issued (``:93``).  ``splits_per_rank`` (default 1) chunks per
    shard; the remaining tile-size kwargs are accepted and ignored.

    fp8 operands (``torch.float8_e4m3fn`` for the shards and ``b``) give an fp8 ``c``
    like in the reference (``:53,121,213``): fp32 accumulate, one rounding to fp8
    (nearest even, magnitudes of 448 and more saturate to 448), in both modes.
    With M and N multiples of 256 and K of 128 the product runs on the fp8
    matrix-core instruction; other sizes (multiples of 16) are widened to bf16 by one
    conversion pass per operand (exact: every e4m3 value is a bf16 value), multiplied
    by the bf16 kernels with an fp32 result and rounded to fp8 by a third pass, after
    the gather has finished.  ``a_gathered`` stays fp8.
    """
    fp8 = torch.float8_e4m3fn
    peers = PeerBuffers(a_shared, dtypes=(torch.bfloat16, fp8))
    if peers.slice(0).dtype == fp8:
        return _all_gather_matmul_fp8(a_shared, peers, b, a_out, progress, **kwargs)
    W = peers.W
    shard = peers.slice(0)
    assert shard.dim() == 2, "expected shards of shape [m, K]"
    assert b.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    m, K = shard.shape
    assert b.dim() == 2 and b.shape[0] == K
    if not b.T.is_contiguous():
        raise ValueError("b.T must be contiguous")
    rank = kwargs.get("rank", 0)
    assert 0 <= rank < W
    splits = kwargs.get("splits_per_rank", 1)
    M, N = W * m, b.shape[1]
    assert N % 8 == 0, "N must be a multiple of 8"
    stacked = peers.stacked is not None and peers.stacked.is_contiguous()
    gather = kwargs.get("gather", not stacked)
    dev = _lib.require_device(*peers.tensors, b, a_out, progress)

    if not gather:
        assert stacked, "gather=False needs the shards as one contiguous [W, m, K] tensor"
        a_full = peers.stacked.reshape(M, K)
        if a_out is not None:
            assert a_out.shape == a_full.shape and a_out.dtype == a_full.dtype
            a_out.copy_(a_full)
        else:
            a_out = a_full
        if progress is not None:
            progress.fill_(1)
        a2, b2 = _gemm.prepare_operands(a_full, b)
        c = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        _gemm.launch("all_gather_matmul", a2, b2, M, N, None, 0, 0, None, 0, M, None, c, rank * m)
        return a_out, c

    assert K % 8 == 0, "K must be a multiple of 8"
    assert m % splits == 0, "splits_per_rank must divide the rows of a shard"
    _waits.check()      # an earlier call's failed wait is reported before anything of this call is enqueued
    if a_out is None:
        a_out = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
    else:
        assert tuple(a_out.shape) == (M, K) and a_out.dtype == torch.bfloat16 and a_out.is_contiguous()
    if progress is None:
        progress = torch.zeros(W * splits, dtype=torch.int32, device=dev)
    else:
        progress.fill_(0)
    backend_stream = _copy_engine_all_gather_w_progress(a_out, a_shared, progress, splits, rank=rank,
                                                        copy_engine=kwargs.get("copy_engine", False))
    configs = {"RANK": rank, "WORLD_SIZE": W, "SPLITS_PER_RANK": splits,
               "wait_limit_us": kwargs.get("wait_limit_us", 0)}
    status = kwargs.get("status")
    own_status = status is None
    if own_status:
        status = _waits.new_status(dev)
    c = _matmul_w_progress(a_out, peers.slice(rank), b, progress, configs, status)
    torch.cuda.current_stream(dev).wait_stream(backend_stream)
    if own_status:
        _waits.watch(status, "all_gather_matmul")
    return a_out, c
