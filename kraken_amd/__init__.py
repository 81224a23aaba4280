"""kraken_amd — the one-rank arithmetic of Kraken's fused comm+compute kernels on AMD MI355X.

Mirrors the public layout of the reference package (``kraken/__init__.py:1-13``):
``kraken_amd.comm`` and ``kraken_amd.fused`` export the same function names with
the same argument order.  Where the reference takes a symmetric-memory tensor
(or an implicit symmetric-memory workspace) that stands for the W peers'
buffers, these functions take one device tensor of shape ``[W, ...]`` whose W
slices are the peers' buffers.  All arithmetic runs in hand-written gfx950 HIP
kernels behind the C ABI declared in ``include/kraken_amd.h``; there is no CPU
or eager-PyTorch fallback — a missing library or a non-HIP tensor raises.
"""
from . import _lib, _logging, comm, fused

__all__ = ["_lib", "_logging", "comm", "fused"]
__version__ = "0.1.0"
