"""Shared argument handling of the W-way reduce wrappers."""
from __future__ import annotations

import torch

from .. import _lib


def check_stack(stacked: torch.Tensor) -> tuple[int, int, int]:
    """Validate a ``[W, ...]`` stack; return (W, slice_capacity, slice_stride) in elements.

    Mirrors the dtype/alignment asserts of ``kraken/comm/one_shot_all_reduce.py:79-80``.
    """
    assert stacked.dim() >= 2, "expected a stacked tensor of shape [W, ...]"
    assert stacked.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    W = stacked.shape[0]
    assert W >= 1
    assert stacked[0].is_contiguous(), "each of the W slices must be contiguous"
    cap = stacked[0].numel()
    stride = stacked.stride(0) if W > 1 else cap
    return W, cap, stride


def stage_input(stacked: torch.Tensor, input_tensor: torch.Tensor | None, rank: int) -> None:
    """Copy ``input_tensor`` into slice ``rank`` of the stack.

    Stands in for the copy-in stage of the reference kernels
    (``kraken/fused/one_shot_all_reduce_bias.py:56-65``).  Skipped when the
    tensor already is (a prefix of) that slice.
    """
    if input_tensor is None:
        return
    n = input_tensor.numel()
    dst = stacked[rank].reshape(-1)[:n]
    if dst.data_ptr() == input_tensor.data_ptr():
        return
    dst.copy_(input_tensor.reshape(-1))


def bias_args(bias: torch.Tensor | None, numel: int, D: int) -> tuple[int | None, int]:
    """Return (pointer, bias_numel) for a bias of the input's shape or of shape [D]."""
    if bias is None:
        return None, 0
    assert bias.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    assert bias.is_contiguous()
    assert bias.numel() in (numel, D), (
        f"bias must have the shape of the input ({numel} elements) or be a vector of the last dim ({D})"
    )
    return _lib.ptr(bias), bias.numel()
