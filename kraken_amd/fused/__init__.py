"""Mirror of ``kraken/fused/__init__.py:1-27``: same names, same argument order."""
from .all_gather_matmul import all_gather_matmul
from .gemm_one_shot_all_reduce_fused import (
    gemm_one_shot_all_reduce as gemm_one_shot_all_reduce_fused,
)
from .gemm_reduce_scatter_ce_persistent import gemm_reduce_scatter_ce_persistent
from .gemm_reduce_scatter_fused import gemm_reduce_scatter
from .one_shot_all_reduce_bias import one_shot_all_reduce_bias
from .one_shot_all_reduce_bias_rms_norm import one_shot_all_reduce_bias_rms_norm
from .rms_norm import rms_norm
from .two_shot_all_reduce_bias import two_shot_all_reduce_bias
from .two_shot_all_reduce_bias_rms_norm import two_shot_all_reduce_bias_rms_norm

__all__ = [
    "all_gather_matmul",
    "gemm_one_shot_all_reduce_fused",
    "gemm_reduce_scatter",
    "gemm_reduce_scatter_ce_persistent",
    "one_shot_all_reduce_bias",
    "one_shot_all_reduce_bias_rms_norm",
    "rms_norm",
    "two_shot_all_reduce_bias",
    "two_shot_all_reduce_bias_rms_norm",
]
