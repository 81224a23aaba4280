"""Mirror of ``kraken/comm/__init__.py:1-17``: same names."""
from .copy_engine_all_gather import _copy_engine_all_gather_w_progress, all_gather_w_progress
from .one_shot_all_reduce import one_shot_all_reduce
from .two_shot_all_reduce import two_shot_all_reduce

__all__ = [
    "_copy_engine_all_gather_w_progress",
    "all_gather_w_progress",
    "one_shot_all_reduce",
    "two_shot_all_reduce",
]
