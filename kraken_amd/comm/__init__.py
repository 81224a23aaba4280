"""Mirror of ``kraken/comm/__init__.py:1-17`` (the reduce entry points).

``all_gather_w_progress`` / ``_copy_engine_all_gather_w_progress`` of the
reference move data between GPUs with copy engines and compute nothing; on
one GPU the gathered operand is the ``[W, m, K]`` stack itself, so they have no
counterpart here.
"""
from .one_shot_all_reduce import one_shot_all_reduce
from .two_shot_all_reduce import two_shot_all_reduce

__all__ = ["one_shot_all_reduce", "two_shot_all_reduce"]
