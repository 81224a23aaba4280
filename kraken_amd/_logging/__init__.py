from .benchmarking import benchmark_with_event

__all__ = ["benchmark_with_event"]
