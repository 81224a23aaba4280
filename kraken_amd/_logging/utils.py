"""Plot of a sweep's running times (``kraken/_logging/utils.py:27-61``)."""
from __future__ import annotations


def plot_experiment_comparison(sizes: list[str], experiments: list[str], data: list[list[float]], filename: str) -> None:
    """Line chart of running time (microseconds) against input size, one line per experiment.

    ``data[i][j]`` is the time of ``experiments[j]`` at ``sizes[i]``; the chart is written to
    ``filename``.  Needs matplotlib (imported here, so that nothing else depends on it).
    """
    import matplotlib

    matplotlib.use("Agg")
    from matplotlib import pyplot

    assert len(data) == len(sizes) and all(len(row) == len(experiments) for row in data)
    fig, ax = pyplot.subplots(figsize=(12, 6))
    xs = list(range(len(sizes)))
    for j, name in enumerate(experiments):
        ax.plot(xs, [row[j] for row in data], marker="o", label=name)
    ax.set_xticks(xs)
    ax.set_xticklabels(sizes, rotation=30, ha="right")
    ax.set_xlabel("Sizes")
    ax.set_ylabel("Running Time (us)")
    ax.set_title("Experiments")
    ax.grid(True, axis="y")
    ax.legend()
    fig.tight_layout()
    fig.savefig(filename, dpi=300)
    pyplot.close(fig)
    print(f"Plot saved as {filename}")
