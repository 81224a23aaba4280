from .benchmarking import benchmark_with_event, benchmark_with_profiler
from .utils import plot_experiment_comparison

__all__ = ["benchmark_with_event", "benchmark_with_profiler", "plot_experiment_comparison"]
