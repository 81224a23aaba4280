"""Two-shot all-reduce + bias, local arithmetic (``kraken/fused/two_shot_all_reduce_bias.py``)."""
from __future__ import annotations

import torch

from .. import _lib
from ..comm._common import bias_args, check_stack, stage_input


def two_shot_all_reduce_bias(
    symm_mem_input,
    input_tensor: torch.Tensor | None,
    bias: torch.Tensor | None,
    output: torch.Tensor,
    max_num_blocks: int = 24,
    BLOCK_SIZE: int = 2048,
    group=None,
    *,
    rank: int = 0,
    stage: bool = False,
    layout: str = "rows",
    numel: int | None = None,
) -> torch.Tensor:
    """Two-shot order: ``sum over slices 0..W-1`` from 0.0, bias added last (fp32).

    Counterpart of ``kraken.fused.two_shot_all_reduce_bias``
    (``kraken/fused/two_shot_all_reduce_bias.py:123-193``; arithmetic ``:66-83``).
    The size of ``output`` selects what is computed:

    * ``output.numel() == message numel``: all W shares, i.e. the full
      all-reduced tensor (what the reference returns after its broadcast step);
    * otherwise ``output`` receives only the share of rank ``rank``:
      ``layout="rows"`` — contiguous chunk ``rank`` of ``numel/W`` elements;
      ``layout="striped"`` — the reference's interleaved ownership with stripe
      block ``BLOCK_SIZE`` (``:66-69``), written compactly.

    ``symm_mem_input`` is the ``[W, ...]`` stack or a list of W separate
    tensors.  The message length is ``input_tensor.numel()`` if an input is given
    (it is read in place as rank ``rank``'s contribution; ``stage=True`` also
    copies it into slice ``rank`` first, the reference's copy-in ``:43-50``), else ``numel`` if passed, else ``bias.numel()`` for a
    full-shape bias, else the slice size.  Returns ``output``.
    """
    peers = check_stack(symm_mem_input)
    W, cap = peers.W, peers.cap
    assert BLOCK_SIZE % W == 0
    assert layout in ("rows", "striped")
    assert 0 <= rank < W
    if input_tensor is not None:
        assert input_tensor.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
        n = input_tensor.numel()
    elif numel is not None:
        n = int(numel)
    elif output.numel() == cap or output.numel() * W == cap:
        n = cap
    else:
        n = output.numel() * W if layout == "rows" else cap
    assert n % 8 == 0, "The number of elements must be 128-bit aligned."
    assert n <= cap, "the message does not fit in one slice of the stacked buffer"
    assert output.dtype == torch.bfloat16 and output.is_contiguous()
    ref = input_tensor if input_tensor is not None else peers.slice(0)
    D = ref.shape[-1]
    if bias is not None:
        assert bias.dtype == torch.bfloat16 and bias.is_contiguous()
    dev = _lib.require_device(*peers.tensors, input_tensor, bias, output)
    peers = stage_input(peers, input_tensor, rank, stage)
    lib = _lib.load()
    stream = _lib.current_stream(dev)

    if output.numel() == n:  # every share: the full result
        bias_ptr, bias_numel = bias_args(bias, n, D)
        rc = peers.reduce(0, n, bias_ptr, bias_numel, D, 0, output.data_ptr(), stream)
        _lib.check(rc, "two_shot_all_reduce_bias")
        return output

    if layout == "striped":
        share = lib.kr_striped_share_numel(n, W, BLOCK_SIZE, rank)
        _lib.check(min(share, 0), "two_shot_all_reduce_bias")
        assert output.numel() == share, f"output must hold the {share} elements rank {rank} owns"
        if bias is not None:
            assert bias.numel() == n, "striped ownership needs a bias of the input's shape"
        rc = peers.reduce_striped(n, _lib.ptr(bias), BLOCK_SIZE, rank, output.data_ptr(), stream)
        _lib.check(rc, "two_shot_all_reduce_bias")
        return output

    assert n % W == 0, "the number of elements must be divisible by the world size"
    share = n // W
    assert share % 8 == 0, "each rank's share must be 128-bit aligned"
    assert output.numel() == share, f"output must hold numel/W = {share} elements (or the full {n})"
    off = rank * share
    bias_ptr, bias_numel = None, 0
    if bias is not None:
        if bias.numel() == n:
            bias_ptr, bias_numel = bias.data_ptr() + 2 * off, share
        else:
            assert bias.numel() == D and share % D == 0, "a vector bias needs shares made of whole rows"
            bias_ptr, bias_numel = bias.data_ptr(), D
    rc = peers.reduce(off, share, bias_ptr, bias_numel, D, 0, output.data_ptr(), stream)
    _lib.check(rc, "two_shot_all_reduce_bias")
    return output
