"""Stand-alone RMSNorm (``kraken/fused/rms_norm.py``)."""
from __future__ import annotations

import math

import torch

from .. import _lib


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float = 1.0e-5) -> torch.Tensor:
    """``y = x * rsqrt(mean(x^2, -1) + eps) * w`` in fp32, rounded to bf16 once.

    Counterpart of ``kraken.fused.rms_norm`` (``kraken/fused/rms_norm.py:46-72``;
    arithmetic ``:34-43``).
    """
    D = x.shape[-1]
    assert w.is_contiguous()
    assert w.shape == (D,)
    assert x.is_contiguous()
    assert x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "Only bfloat16 is supported for now."
    assert D % 8 == 0, "The row length must be 128-bit aligned."
    dev = _lib.require_device(x, w)
    y = torch.empty_like(x)
    rows = math.prod(x.shape[:-1])
    rc = _lib.load().kr_rmsnorm_bf16(
        x.data_ptr(), w.data_ptr(), float(eps), rows, D, y.data_ptr(), _lib.current_stream(dev)
    )
    _lib.check(rc, "rms_norm")
    return y
