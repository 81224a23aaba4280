"""Shape sweeps with backend tables, after the reference's ``benchmark/benchmark_*.py``.

One GPU holds all W ranks' buffers, so the "backends" compared are what one
GPU can run on the same inputs: this library's kernels and plain PyTorch
(eager ops; its matmul is hipBLASLt).  As in the reference the first backend
given is the baseline: every other backend is checked against its output,
timed with ``benchmark_with_event`` (caches flushed before every call), and
the table reports the time of each backend in microseconds, the speed-up of
the best one over the baseline and which one was best; ``save_path`` writes
the same table as CSV (``benchmark/benchmark_all_reduce.py:158-190``).
"""
from __future__ import annotations

import csv
from collections import defaultdict
from typing import Callable

import torch

from .. import comm, fused
from .benchmarking import benchmark_with_event

BF16 = torch.bfloat16


def _fmt(num: int) -> str:
    for sh, suffix in ((30, "g"), (20, "m"), (10, "k")):
        if num >= 1 << sh and num % (1 << sh) == 0:
            return f"{num >> sh}{suffix}"
    return str(num)


def _randn(shape, dev, seed, std=1.0):
    g = torch.Generator(device=dev).manual_seed(seed)
    return (torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * std).to(BF16)


# ---- all-reduce (benchmark/benchmark_all_reduce.py) ---------------------------------------
def _all_reduce_case(size: int, W: int, dev) -> dict[str, Callable[[], torch.Tensor]]:
    stack = _randn((W, size), dev, 42)
    return {
        "hip_1shot": lambda: comm.one_shot_all_reduce(stack),
        "hip_2shot": lambda: comm.two_shot_all_reduce(stack, rank=None),
        "torch": lambda: stack.sum(0, dtype=torch.float32).to(BF16),
    }


# ---- all-reduce + bias (benchmark/benchmark_all_reduce_bias.py) ---------------------------
def _all_reduce_bias_case(shape, W: int, dev):
    b, d = shape
    stack = _randn((W, b, d), dev, 42 + b)
    bias = _randn((b, d), dev, 42)
    out = torch.empty(b, d, dtype=BF16, device=dev)

    def one():
        fused.one_shot_all_reduce_bias(stack, None, bias, out)
        return out

    def two():
        return fused.two_shot_all_reduce_bias(stack, None, bias, out)

    return {"hip_1shot": one, "hip_2shot": two,
            "torch": lambda: (stack.sum(0, dtype=torch.float32) + bias.float()).to(BF16)}


# ---- all-reduce + bias + RMSNorm (benchmark/benchmark_all_reduce_bias_rms_norm.py) --------
def _all_reduce_bias_rms_norm_case(shape, W: int, dev):
    b, d = shape
    stack = _randn((W, b, d), dev, 42 + b)
    bias = _randn((b, d), dev, 42)
    w = _randn((d,), dev, 43)
    y = torch.empty(b, d, dtype=BF16, device=dev)

    def one():
        fused.one_shot_all_reduce_bias_rms_norm(stack, None, bias, w, y)
        return y

    def unfused():     # the reduce + bias kernel, then the stand-alone norm kernel
        fused.one_shot_all_reduce_bias(stack, None, bias, y)
        return fused.rms_norm(y, w, 1e-5)

    def eager():
        s = stack.sum(0, dtype=torch.float32) + bias.float()
        return torch.nn.functional.rms_norm(s, (d,), w.float(), 1e-5).to(BF16)

    return {"hip_fused": one, "hip_unfused": unfused, "torch": eager}


# ---- GEMM + reduce-scatter (benchmark/benchmark_matmul_reduce_scatter.py) ------------------
def _matmul_reduce_scatter_case(shape, W: int, dev):
    M, N, K = shape
    a = _randn((M, K), dev, 42)
    b = _randn((N, K), dev, 43, 0.02).T
    peers = _randn((W - 1, M // W, N), dev, 44)
    c = torch.empty(M, N, dtype=BF16, device=dev)

    def eager():
        full = a @ b
        return (full[: M // W].float() + peers.sum(0, dtype=torch.float32)).to(BF16)

    return {
        "hip": lambda: fused.gemm_reduce_scatter(a, b, peers=peers, rank=0, c_scratch=c),
        "hip_ce": lambda: fused.gemm_reduce_scatter_ce_persistent(a, b, peers=peers, rank=0, world_size=W),
        "torch": eager,
    }


# ---- all-gather + matmul (benchmark/benchmark_all_gather_matmul.py) ------------------------
def _all_gather_matmul_case(shape, W: int, dev):
    M, N, K = shape          # M = rows of one rank's shard, as in the reference's sweep
    stack = _randn((W, M, K), dev, 42)
    shards = [stack[r].clone() for r in range(W)]
    b = _randn((N, K), dev, 43, 0.02).T
    a_out = torch.empty(W * M, K, dtype=BF16, device=dev)
    return {
        "hip": lambda: fused.all_gather_matmul(stack, b)[1],
        "hip_overlap": lambda: fused.all_gather_matmul(shards, b, a_out=a_out)[1],
        "torch": lambda: torch.cat(shards) @ b,
    }


def _pow2(lo: int, hi: int) -> list[int]:
    return [1 << k for k in range(lo, hi + 1)]


SWEEPS = {
    # name: (case builder, default shapes, tolerance of the cross-check)
    "all_reduce": (_all_reduce_case, [1 << k for k in range(12, 27, 2)], 1e-1),
    "all_reduce_bias": (_all_reduce_bias_case, [(b, 5120) for b in _pow2(0, 9)], 5e-2),
    "all_reduce_bias_rms_norm": (_all_reduce_bias_rms_norm_case, [(b, 5120) for b in _pow2(0, 9)], 5e-2),
    "matmul_reduce_scatter": (_matmul_reduce_scatter_case,
                              [(m, 6656, k) for m in _pow2(7, 10) for k in _pow2(12, 15)], 5e-2),
    "all_gather_matmul": (_all_gather_matmul_case,
                          [(m, 6656, k) for m in _pow2(7, 10) for k in _pow2(12, 15)], 5e-2),
}


def run_sweep(name: str, backends: list[str] | None = None, shapes=None, world_size: int = 8,
              save_path: str | None = None, iters: int = 25, dev=None, plot_path: str | None = None) -> list[dict]:
    """Run sweep ``name``; print the table; return one dict per shape.  ``plot_path``: also
    draw the times against the shapes, one line per backend, as the reference's bias sweeps do
    (``benchmark/benchmark_all_reduce_bias.py:150-154``)."""
    from tabulate import tabulate

    build, default_shapes, tol = SWEEPS[name]
    dev = dev or torch.device("cuda:0")
    rows = []
    for shape in shapes or default_shapes:
        fns = build(shape, world_size, dev)
        order = backends or list(fns)
        for be in order:
            if be not in fns:
                raise ValueError(f"sweep {name} has no backend '{be}' (choices: {', '.join(fns)})")
        golden = fns[order[0]]().float()
        row = {"shape": "(" + ", ".join(_fmt(int(s)) for s in (shape if isinstance(shape, tuple) else (shape,))) + ")",
               "dtype": "bfloat16", "world_size": world_size}
        for be in order:
            got = fns[be]().float()
            torch.testing.assert_close(got, golden, atol=tol * max(1.0, golden.abs().max().item() / 4), rtol=tol)
            row[be] = benchmark_with_event(lambda i, f=fns[be]: f(), warmup_iters=10, benchmark_iters=iters,
                                           flush_bytes=1 << 29)
        best = min(order, key=lambda be: row[be])
        row[f"Speedup over {order[0]}"] = row[order[0]] / row[best]
        row["Best Backend"] = best
        rows.append(row)
        del fns, golden
        torch.cuda.empty_cache()
    table = defaultdict(list)
    for row in rows:
        for k, v in row.items():
            table[k].append(v)
    print(tabulate(table, headers="keys", tablefmt="github", floatfmt=".3f"))
    if plot_path is not None:
        from .utils import plot_experiment_comparison

        names = backends or [k for k in rows[0] if k not in ("shape", "dtype", "world_size", "Best Backend")
                             and not k.startswith("Speedup")]
        plot_experiment_comparison([r["shape"] for r in rows], names, [[r[b] for b in names] for r in rows], plot_path)
    if save_path is not None:
        with open(save_path, "w", newline="") as f:
            wr = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
            wr.writeheader()
            wr.writerows(rows)
        print(f"\nResults saved to {save_path}")
    return rows
