"""Shared host logic of the GEMM + reduce wrappers."""
from __future__ import annotations

import ctypes

import torch

from .. import _lib


def split_fp32(a: torch.Tensor, b: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """fp32 operands for the bf16 matrix cores: a = a_hi + a_lo, b = b_hi + b_lo.

    ``[a_hi | a_hi | a_lo] @ [b_hi ; b_lo ; b_hi]`` (one GEMM with 3K inner
    length, fp32 accumulate) equals ``a@b`` up to the dropped ``a_lo@b_lo``
    term, i.e. about 16 mantissa bits — tighter than the TF32 ``tl.dot`` the
    reference runs fp32 inputs through (``gemm_one_shot_all_reduce_fused.py:56-64``).
    Each operand is split in one pass of ``kr_split_fp32`` over it (read fp32 once,
    write the three bf16 blocks); operands whose layout that kernel does not take
    (K or N not a multiple of 8, a column-major left operand, rows not 16-byte
    aligned) are made contiguous first, or, for odd sizes, split by elementwise torch ops.
    """
    M, K = a.shape
    N = b.shape[1]
    if not (a.is_cuda and b.is_cuda) or K % 8 != 0 or N % 8 != 0:
        a_hi = a.to(torch.bfloat16)
        a_lo = (a - a_hi.float()).to(torch.bfloat16)
        b_hi = b.to(torch.bfloat16)
        b_lo = (b - b_hi.float()).to(torch.bfloat16)
        return torch.cat([a_hi, a_hi, a_lo], dim=1), torch.cat([b_hi, b_lo, b_hi], dim=0)
    lib = _lib.load()
    dev = _lib.require_device(a, b)
    stream = _lib.current_stream(dev)

    def rows_ok(t):      # columns contiguous, rows 16-byte aligned
        return t.stride(1) == 1 and t.stride(0) % 4 == 0 and t.stride(0) >= t.shape[1] and t.data_ptr() % 16 == 0

    if not rows_ok(a):
        a = a.contiguous()
    a3 = torch.empty((M, 3 * K), dtype=torch.bfloat16, device=dev)
    _lib.check(lib.kr_split_fp32(a.data_ptr(), M, K, a.stride(0), 1, 0, a3.data_ptr(), 3 * K, stream), "split_fp32(a)")
    if rows_ok(b.T) and not rows_ok(b):
        # transposed-contiguous right operand: memory is [N, K]; the blocks lie side by side along K
        bt = b.T
        b3t = torch.empty((N, 3 * K), dtype=torch.bfloat16, device=dev)
        _lib.check(lib.kr_split_fp32(bt.data_ptr(), N, K, bt.stride(0), 1, 1, b3t.data_ptr(), 3 * K, stream), "split_fp32(b)")
        return a3, b3t.T
    if not rows_ok(b):
        b = b.contiguous()
    b3 = torch.empty((3 * K, N), dtype=torch.bfloat16, device=dev)
    _lib.check(lib.kr_split_fp32(b.data_ptr(), K, N, b.stride(0), 0, 1, b3.data_ptr(), N, stream), "split_fp32(b)")
    return a3, b3


def prepare_operands(a: torch.Tensor, b: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Return bf16 operands in a layout the kernel reads directly.

    A must be k-contiguous; B either row-major or transposed-contiguous; any row
    stride that is a multiple of 8 elements is read in place (the kernels address
    operands through buffer descriptors built from the caller's strides).  Other
    stridings (the reference accepts any 2-D strides,
    ``gemm_one_shot_all_reduce_fused.py:163-166``) take one copy.  fp32 operands are
    split into bf16 parts by one kernel pass each (``split_fp32``).
    K is padded to a multiple of 8 with zeros when necessary.
    """
    assert a.dim() == 2 and b.dim() == 2
    assert a.shape[1] == b.shape[0], "Inner dimensions must match for matrix multiplication"
    assert a.dtype == b.dtype, "Input tensors must have the same dtype"
    assert a.dtype in (torch.bfloat16, torch.float32), "bfloat16 (or float32) operands expected"
    if a.dtype == torch.float32:
        a, b = split_fp32(a, b)
    K = a.shape[1]
    if K % 8 != 0:
        pad = 8 - K % 8
        a = torch.nn.functional.pad(a, (0, pad))
        b = torch.nn.functional.pad(b, (0, 0, 0, pad))
    if a.stride(1) != 1 or a.stride(0) % 8 != 0 or a.data_ptr() % 16 != 0:
        a = a.contiguous()
    b_ok = (b.stride(1) == 1 and b.stride(0) % 8 == 0) or (b.stride(0) == 1 and b.stride(1) % 8 == 0)
    if not b_ok or b.data_ptr() % 16 != 0:
        b = b.contiguous()
    return a, b


_workspaces: dict[tuple[int, int], torch.Tensor] = {}


def workspace(dev: torch.device, nbytes: int) -> torch.Tensor | None:
    """Scratch for the split K loop, one buffer per (device, stream), grown on demand (a
    buffer per stream keeps calls on different streams from sharing one)."""
    if nbytes <= 0:
        return None
    key = (dev.index if dev.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(dev).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
        _workspaces[key] = ws
    return ws


def launch(name, a, b, M, N, peers, n_peers, peers_stride, bias, band_row0, band_rows, c_full, out, pivot):
    """One call of the GEMM entry point; ``peers`` is a ``[P, rows, N]`` tensor (stacked entry
    point), a list of P tensors (pointer-table entry point) or ``None``.  Shapes with few
    output tiles get a workspace and go through the ``_ws`` entry points (split K loop)."""
    lib = _lib.load()
    out_fp32 = int(out is not None and out.dtype == torch.float32)
    ws = workspace(a.device, lib.kr_gemm_workspace_bytes(M, N, a.shape[1])) if a.is_cuda else None
    if ws is not None:
        if isinstance(peers, (list, tuple)):
            dev = _lib.require_device(a, b, *peers, bias, c_full, out)
            table = (ctypes.c_void_p * max(n_peers, 1))(*[t.data_ptr() for t in peers])
            rc = lib.kr_gemm_reduce_ptrs_ws_bf16(
                a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1),
                M, N, a.shape[1], table, n_peers, _lib.ptr(bias), band_row0, band_rows, _lib.ptr(c_full),
                _lib.ptr(out), out_fp32, pivot, ws.data_ptr(), ws.numel(), _lib.current_stream(dev),
            )
        else:
            dev = _lib.require_device(a, b, peers, bias, c_full, out)
            rc = lib.kr_gemm_reduce_ws_bf16(
                a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1),
                M, N, a.shape[1], _lib.ptr(peers), n_peers, peers_stride, _lib.ptr(bias), band_row0, band_rows,
                _lib.ptr(c_full), _lib.ptr(out), out_fp32, pivot, ws.data_ptr(), ws.numel(),
                _lib.current_stream(dev),
            )
        _lib.check(rc, name)
        return
    if isinstance(peers, (list, tuple)):
        dev = _lib.require_device(a, b, *peers, bias, c_full, out)
        table = (ctypes.c_void_p * max(n_peers, 1))(*[t.data_ptr() for t in peers])
        rc = lib.kr_gemm_reduce_ptrs_bf16(
            a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1),
            M, N, a.shape[1], table, n_peers, _lib.ptr(bias),
            band_row0, band_rows, _lib.ptr(c_full), _lib.ptr(out), out_fp32, pivot, _lib.current_stream(dev),
        )
    else:
        dev = _lib.require_device(a, b, peers, bias, c_full, out)
        rc = lib.kr_gemm_reduce_bf16(
            a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1),
            M, N, a.shape[1], _lib.ptr(peers), n_peers, peers_stride, _lib.ptr(bias),
            band_row0, band_rows, _lib.ptr(c_full), _lib.ptr(out), out_fp32, pivot, _lib.current_stream(dev),
        )
    _lib.check(rc, name)


def n_peers_of(peers) -> int:
    """Number of pre-staged partials in a ``peers`` argument (tensor, sequence or ``None``)."""
    if peers is None:
        return 0
    return len(peers) if isinstance(peers, (list, tuple)) else peers.shape[0]


def check_peers(peers, rows: int, N: int) -> tuple[int, int]:
    """Validate pre-staged partials — one ``[P, rows, N]`` tensor or a sequence of P
    ``[rows, N]`` tensors (separate allocations); return (P, stride), stride 0 for a sequence."""
    if peers is None:
        return 0, 0
    if isinstance(peers, (list, tuple)):
        for t in peers:
            assert t.dtype == torch.bfloat16, "pre-staged partials must be bfloat16"
            assert tuple(t.shape) == (rows, N) and t.is_contiguous(), (
                f"every peer must be a contiguous [{rows}, {N}] tensor, got {tuple(t.shape)}"
            )
        return len(peers), 0
    assert peers.dtype == torch.bfloat16, "pre-staged partials must be bfloat16"
    assert peers.dim() == 3 and tuple(peers.shape[1:]) == (rows, N), (
        f"peers must have shape [W-1, {rows}, {N}], got {tuple(peers.shape)}"
    )
    assert peers[0].is_contiguous()
    P = peers.shape[0]
    return P, (peers.stride(0) if P > 1 else rows * N)
