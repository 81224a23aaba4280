#!/usr/bin/env python3
"""Benchmark of the one-rank hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all]

A "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM.  The default workload is the configuration the
headline metric is quoted on: the pure one-shot W-way reduce, bf16
[8,4096,4096] -> [4096,4096] (HBM-bound).  One JSON line is printed; with
``--all`` (default) the line also carries, under "configs", the other
benchmark configurations (reduce+bias+RMSNorm, two-shot share, decode shape,
GEMM + reduce-scatter, GEMM + fused all-reduce, all-gather matmul), each
checked against the CPU oracle before it is timed.

Timing: W untimed warm-up steps, then exactly K steps between two device
synchronisations; events recorded on the launch stream around the same K
steps give the average kernel duration used for the roofline figure.  Every
workload rotates several complete operand sets (inputs, peers and outputs,
the GEMM operands A and B included), together larger than the 256 MB
last-level cache, so no step finds its operands cached.  Each entry states
the target the benchmark definition gives for it (a fraction of the HBM or
bf16 matrix-core peak) and whether the measured figure meets it.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
W = 8

# HBM-side bytes per launch of the dominant kernel (L2 fills + write-backs), from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of `bench.py --only --no-cpu --workload <key>`, each counter scaled by
# what it reads for a plain 256 MiB device copy (`bench.py --calibrate-copy`).  bench.py cannot read
# hardware counters itself; the figures and the commands behind them are kept as text under
# profiles/ (one file per kernel and workload).  None: not measured.
MEASURED_TRAFFIC = {
    "one_shot_reduce_w8_4096x4096": 302053204,              # profiles/reduce_kernel_w8_4096x4096.md
    "two_shot_share_w8_512x4096": 37839283,                 # profiles/reduce_kernel_w8_two_shot_share_512x4096.md
    "reduce_bias_rmsnorm_w8_256x4096": 19050022,            # profiles/reduce_rmsnorm_kernel_w8_256x4096.md
    "reduce_bias_rmsnorm_w8_16x8192_decode": 2483922,       # profiles/reduce_rmsnorm_split_kernel_w8_16x8192.md
    "reduce_bias_rmsnorm_w8_16384x4096_large": 1208025963,  # profiles/reduce_rmsnorm_kernel_w8_16384x4096.md
    # the GEMMs: L2 fills (A and B panels re-read per tile row / column, served mostly by the 256 MB
    # last-level cache, not by HBM) + write-backs
    "gemm_reduce_scatter_8192x8192x3584_w8": 962243626,     # profiles/gemm_dtl16_kernel_reduce_scatter_8192x8192x3584.md
    "gemm_all_reduce_4096x8192x1024_w8": 705354977,         # profiles/gemm_dtl_kernel_all_reduce_4096x8192x1024.md
    "all_gather_matmul_8192x3584x8192_w8": 875039914,       # profiles/gemm_dtl16_kernel_all_gather_matmul_8192x3584x8192.md
}

# Targets of the benchmark definition: fraction of the binding roof.  The W = 8 reduce(+bias+RMSNorm)
# paths: 75 % of peak HBM bandwidth; the GEMM + reduce paths at the Llama-70B TP8 shard shapes: 60 %
# of the dense bf16 matrix-core peak.  The decode shape is latency-bound (reported in microseconds
# beside the launch floor) and the fused GEMM + all-reduce is HBM-bound (122 flop/B: its matrix-core
# fraction cannot exceed 39 %), so neither has a target of its own.
TARGETS = {
    "one_shot_reduce_w8_4096x4096": ("hbm", 0.75),
    "two_shot_share_w8_512x4096": ("hbm", 0.75),
    "reduce_bias_rmsnorm_w8_256x4096": ("hbm", 0.75),
    "reduce_bias_rmsnorm_w8_16x8192_decode": (None, None),
    "reduce_bias_rmsnorm_w8_16384x4096_large": ("hbm", 0.75),
    "gemm_reduce_scatter_8192x8192x3584_w8": ("mfma", 0.60),
    "gemm_all_reduce_4096x8192x1024_w8": (None, None),
    "all_gather_matmul_8192x3584x8192_w8": ("mfma", 0.60),
}


def _die_multi_gpu(n: int) -> None:
    print(
        f"bench.py: --gpus {n} is not supported: this build covers the compute of ONE rank on ONE GPU "
        "(the W peer buffers are slices of one HBM tensor); run with --gpus 1.",
        file=sys.stderr,
    )
    sys.exit(2)


# --------------------------------------------------------------------------------------
# workloads
# --------------------------------------------------------------------------------------
class Workload:
    name = ""
    bound = "hbm"          # roofline that binds
    dtype = "bf16 storage, fp32 accumulate"
    bytes = 0              # algorithmic bytes per step
    flops = 0              # algorithmic flop per step
    nsets = 1
    cpu_repeats = 5

    def setup(self, dev):   # allocate device inputs (several rotated sets)
        raise NotImplementedError

    def step(self, i):      # one pass of the hot path (enqueue only)
        raise NotImplementedError

    def check(self):        # compare one pass with the CPU oracle
        raise NotImplementedError

    def cpu_step(self):     # the same pass in the oracle's torch-CPU math
        raise NotImplementedError

    def describe(self):
        return {}


def _rand_sets(shape, nsets, dev, std=1.0, seed=1234):
    import torch

    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    return [(torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * std).to(torch.bfloat16)
            for _ in range(nsets)]


class OneShotReduce(Workload):
    """benchmark config 2: stack [8,4096,4096] -> [4096,4096]."""
    name = "one_shot_reduce_w8_4096x4096"
    R, D = 4096, 4096
    nsets = 4   # 4 x 256 MiB of input: no step finds its input in the 256 MB last-level cache

    def __init__(self):
        self.bytes = (W + 1) * self.R * self.D * 2

    def setup(self, dev):
        import torch
        from oracle import oracle as orc

        self.dev = dev
        self.host = orc.make_stack(W, (self.R, self.D), seed0=42)       # the benchmark inputs, set 0
        self.sets = [self.host.to(dev)] + _rand_sets((W, self.R, self.D), self.nsets - 1, dev)
        self.out = None

    def step(self, i):
        from kraken_amd import comm

        self.out = comm.one_shot_all_reduce(self.sets[i % self.nsets])

    def check(self):
        import torch
        from oracle import oracle as orc

        self.step(0)
        got = self.out.cpu()
        rows = slice(1024, 1024 + 256)
        assert torch.equal(got[rows], orc.reduce(self.host[:, rows])), "one_shot_all_reduce differs from the oracle"
        return "bit-exact vs oracle on rows 1024..1279 of set 0"

    def cpu_step(self):
        from oracle import oracle as orc

        return orc.reduce_library(self.host)

    def describe(self):
        return {"W": W, "shape": [W, self.R, self.D], "out": [self.R, self.D], "kernel": "reduce_kernel"}


class TwoShotShare(OneShotReduce):
    """benchmark config 2, two-shot variant: this rank's 1/8 row chunk [512,4096]."""
    name = "two_shot_share_w8_512x4096"
    nsets = 4
    use_graph = True      # ~6 us kernel: replay the timed steps from a HIP graph

    def __init__(self):
        self.bytes = (W + 1) * (self.R // W) * self.D * 2

    def step(self, i):
        from kraken_amd import comm

        self.out = comm.two_shot_all_reduce(self.sets[i % self.nsets], rank=(i % W))

    def check(self):
        import torch
        from kraken_amd import comm
        from oracle import oracle as orc

        got = comm.two_shot_all_reduce(self.sets[0], rank=3).cpu()
        assert torch.equal(got, orc.reduce(self.host[:, 3 * 512:4 * 512])), "two-shot share differs from the oracle"
        return "bit-exact vs oracle (rank 3 share of set 0)"

    def cpu_step(self):
        from oracle import oracle as orc

        return orc.reduce_library(self.host[:, 3 * 512:4 * 512])


class ReduceBiasRmsNorm(Workload):
    """benchmark configs 1 and 3 (and a large-row variant that fills the GPU)."""

    def __init__(self, rows, D, nsets, tag):
        self.rows, self.D, self.nsets = rows, D, nsets
        self.name = f"reduce_bias_rmsnorm_w8_{rows}x{D}{tag}"
        self.bytes = (W + 1) * rows * D * 2 + 2 * D * 2
        self.cpu_repeats = 7
        self.use_graph = self.bytes < (64 << 20)   # microsecond kernels: time a HIP graph replay

    def setup(self, dev):
        import torch
        from oracle import oracle as orc

        self.dev = dev
        self.host = orc.make_stack(W, (self.rows, self.D), seed0=42)
        self.hbias, self.hw = orc.make_bias_weight(self.D, 42)
        self.sets = [self.host.to(dev)] + _rand_sets((W, self.rows, self.D), self.nsets - 1, dev)
        self.bias, self.w = self.hbias.to(dev), self.hw.to(dev)
        self.y = torch.empty(self.rows, self.D, dtype=torch.bfloat16, device=dev)

    def step(self, i):
        from kraken_amd import fused

        fused.one_shot_all_reduce_bias_rms_norm(self.sets[i % self.nsets], None, self.bias, self.w, self.y, 1e-5)

    def check(self):
        import torch
        from oracle import oracle as orc

        self.step(0)
        rows = slice(0, min(self.rows, 256))
        want = orc.reduce_bias_rms_norm(self.host[:, rows], self.hbias, self.hw, 1e-5)
        torch.testing.assert_close(self.y.cpu()[rows], want, rtol=2e-2, atol=2e-2)
        return "within rtol=atol=2e-2 of the oracle"

    def cpu_step(self):
        from oracle import oracle as orc

        return orc.reduce_bias_rms_norm_library(self.host, self.hbias, self.hw, 1e-5)

    def describe(self):
        from kraken_amd import _lib

        split = _lib.load().kr_rmsnorm_workspace_bytes(W, self.rows, self.D) > 0
        return {"W": W, "shape": [W, self.rows, self.D], "eps": 1e-5,
                "kernel": "reduce_rmsnorm_split_kernel" if split else "reduce_rmsnorm_kernel"}


class GemmReduceScatter(Workload):
    """benchmark config 4: A [8192,3584] @ B [3584,8192]; own 1024-row band + 7 partials."""
    name = "gemm_reduce_scatter_8192x8192x3584_w8"
    bound = "mfma"
    M, N, K = 8192, 8192, 3584
    cpu_repeats = 3
    nsets = 3   # 3 x 386 MB of A, B, peers and outputs in rotation: every step's operands come from HBM

    def __init__(self):
        self.flops = 2 * self.M * self.N * self.K
        self.bytes = (self.M * self.K + self.K * self.N + self.M * self.N + 7 * 1024 * self.N) * 2

    def setup(self, dev):
        import torch
        from oracle import oracle as orc

        self.rank = 3
        self.ha = orc.randn_bf16((self.M, self.K), 42)
        self.hb = orc.randn_bf16((self.K, self.N), 43, 0.02)
        self.hp = torch.stack([orc.randn_bf16((self.M // W, self.N), 100 + j) for j in range(W - 1)])
        self.a = [self.ha.to(dev)] + _rand_sets((self.M, self.K), self.nsets - 1, dev, seed=1)
        self.b = [self.hb.to(dev)] + _rand_sets((self.K, self.N), self.nsets - 1, dev, std=0.02, seed=2)
        self.p = [self.hp.to(dev)] + _rand_sets((W - 1, self.M // W, self.N), self.nsets - 1, dev, seed=3)
        self.c = [torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev) for _ in range(self.nsets)]
        self.out = None

    def step(self, i):
        from kraken_amd import fused

        j = i % self.nsets
        self.out = fused.gemm_reduce_scatter(self.a[j], self.b[j], peers=self.p[j], rank=self.rank, c_scratch=self.c[j])

    def check(self):
        import torch

        self.step(0)
        r0 = self.rank * 1024
        pick = torch.tensor([0, 255, 256, 1023])
        want = self.ha[r0 + pick].float() @ self.hb.float() + self.hp[:, pick].float().sum(0)
        torch.testing.assert_close(self.out.cpu()[pick].float(), want.to(torch.bfloat16).float(), rtol=2e-2, atol=2e-2)
        other = torch.tensor([0, 4096, 8191])   # rows outside the band of rank 3
        torch.testing.assert_close(self.c[0].cpu()[other].float(),
                                   (self.ha[other].float() @ self.hb.float()).to(torch.bfloat16).float(),
                                   rtol=2e-2, atol=2e-2)
        return "sampled rows within rtol=atol=2e-2 of the oracle"

    def cpu_step(self):
        from oracle import oracle as orc

        return orc.gemm_reduce_scatter(self.ha, self.hb, self.hp, self.rank, W)

    def describe(self):
        return {"M": self.M, "N": self.N, "K": self.K, "peers": [7, 1024, self.N], "kernel": "gemm_dtl16_kernel",
                "operand_sets": self.nsets}


class GemmAllReduce(Workload):
    """benchmark config 5 (fused): A [4096,1024] @ B [1024,8192] + 7 partials + bias; HBM-bound."""
    name = "gemm_all_reduce_4096x8192x1024_w8"
    bound = "hbm"
    M, N, K = 4096, 8192, 1024
    cpu_repeats = 3
    nsets = 2

    def __init__(self):
        self.flops = 2 * self.M * self.N * self.K
        self.bytes = (self.M * self.K + self.K * self.N + 8 * self.M * self.N + self.N) * 2

    def setup(self, dev):
        import torch
        from oracle import oracle as orc

        self.ha = orc.randn_bf16((self.M, self.K), 42)
        self.hb = orc.randn_bf16((self.K, self.N), 43, 0.02)
        self.hbias = orc.randn_bf16((self.N,), 42, 0.02)
        self.hp = torch.stack([orc.randn_bf16((self.M, self.N), 100 + j) for j in range(W - 1)])
        self.bias = self.hbias.to(dev)
        self.a = [self.ha.to(dev)] + _rand_sets((self.M, self.K), self.nsets - 1, dev, seed=1)
        self.b = [self.hb.to(dev)] + _rand_sets((self.K, self.N), self.nsets - 1, dev, std=0.02, seed=2)
        self.psets = [self.hp.to(dev)] + _rand_sets((W - 1, self.M, self.N), self.nsets - 1, dev)
        self.out = None

    def step(self, i):
        import torch
        from kraken_amd import fused

        j = i % self.nsets
        self.out = fused.gemm_one_shot_all_reduce_fused(self.a[j], self.b[j], peers=self.psets[j],
                                                        bias=self.bias, out_dtype=torch.bfloat16)

    def check(self):
        import torch

        self.step(0)
        pick = torch.tensor([0, 127, 128, 2048, 4095])
        want = self.ha[pick].float() @ self.hb.float() + self.hp[:, pick].float().sum(0) + self.hbias.float()
        torch.testing.assert_close(self.out.cpu()[pick].float(), want.to(torch.bfloat16).float(), rtol=2e-2, atol=2e-2)
        return "sampled rows within rtol=atol=2e-2 of the oracle"

    def cpu_step(self):
        import torch
        from oracle import oracle as orc

        return orc.gemm_all_reduce(self.ha, self.hb, self.hp, self.hbias, torch.bfloat16)

    def describe(self):
        return {"M": self.M, "N": self.N, "K": self.K, "peers": [7, self.M, self.N], "bias": [self.N],
                "kernel": "gemm_dtl_kernel", "operand_sets": self.nsets}


class AllGatherMatmul(Workload):
    """benchmark config 5 (all-gather): A stack [8,1024,8192] @ B [8192,3584], B.T contiguous."""
    name = "all_gather_matmul_8192x3584x8192_w8"
    bound = "mfma"
    m, K, N = 1024, 8192, 3584
    cpu_repeats = 3
    nsets = 3   # 3 x 252 MB of A shards, B and C in rotation: every step's operands come from HBM

    def __init__(self):
        self.flops = 2 * W * self.m * self.N * self.K
        self.bytes = (W * self.m * self.K + self.K * self.N + W * self.m * self.N) * 2

    def setup(self, dev):
        from oracle import oracle as orc

        self.hs = orc.make_stack(W, (self.m, self.K), seed0=42)
        self.hbT = orc.randn_bf16((self.N, self.K), 43, 0.02)
        self.s = [self.hs.to(dev)] + _rand_sets((W, self.m, self.K), self.nsets - 1, dev, seed=1)
        self.bT = [self.hbT.to(dev)] + _rand_sets((self.N, self.K), self.nsets - 1, dev, std=0.02, seed=2)
        self.c = [None] * self.nsets

    def step(self, i):
        from kraken_amd import fused

        j = i % self.nsets
        self.c[j] = None                         # (the allocator hands this set's own block back)
        _, self.c[j] = fused.all_gather_matmul(self.s[j], self.bT[j].T, rank=3)

    def check(self):
        import torch

        self.step(0)
        pick = torch.tensor([0, 1023, 3072, 8191])
        want = self.hs.reshape(-1, self.K)[pick].float() @ self.hbT.T.float()
        torch.testing.assert_close(self.c[0].cpu()[pick].float(), want.to(torch.bfloat16).float(), rtol=2e-2, atol=2e-2)
        return "sampled rows within rtol=atol=2e-2 of the oracle"

    def cpu_step(self):
        from oracle import oracle as orc

        return orc.all_gather_matmul(self.hs, self.hbT.T)

    def describe(self):
        return {"W": W, "m": self.m, "K": self.K, "N": self.N, "b_layout": "b.T contiguous", "kernel": "gemm_dtl16_kernel",
                "operand_sets": self.nsets}


def make_workloads():
    return {
        "cfg2_one_shot": OneShotReduce,
        "cfg2_two_shot_share": TwoShotShare,
        "cfg1_reduce_bias_rmsnorm": lambda: ReduceBiasRmsNorm(256, 4096, 24, ""),
        "cfg3_decode_reduce_bias_rmsnorm": lambda: ReduceBiasRmsNorm(16, 8192, 160, "_decode"),
        "rows16k_reduce_bias_rmsnorm": lambda: ReduceBiasRmsNorm(16384, 4096, 3, "_large"),
        "cfg4_gemm_reduce_scatter": GemmReduceScatter,
        "cfg5_gemm_all_reduce": GemmAllReduce,
        "cfg5_all_gather_matmul": AllGatherMatmul,
    }


# --------------------------------------------------------------------------------------
# measurement
# --------------------------------------------------------------------------------------
def time_gpu_graph(wl, steps, warmup):
    """Device time per step with the `steps` launches replayed from one HIP graph.

    For workloads whose kernel runs only a few microseconds the host cannot enqueue launches
    as fast as the GPU retires them, and events around an eager loop would measure the host.
    (The reference's benchmark_with_event has the same option, _logging/benchmarking.py:98-108.)
    """
    import torch

    for i in range(warmup):
        wl.step(i)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        wl.step(0)
        with torch.cuda.graph(graph, stream=side):
            for i in range(steps):
                wl.step(warmup + i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    graph.replay()
    end.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, start.elapsed_time(end) / steps


def time_gpu(wl, steps, warmup):
    """Return (wall ms per step, event ms per step) over exactly `steps` steps."""
    import torch

    if getattr(wl, "use_graph", False):
        return time_gpu_graph(wl, steps, warmup)
    for i in range(warmup):
        wl.step(i)
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()                      # on the current stream = the stream the kernels go to
    for i in range(steps):
        wl.step(warmup + i)
    end.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, start.elapsed_time(end) / steps


def time_cpu(wl, budget_s=12.0):
    """Median seconds per pass of the oracle's torch-CPU math for the same workload."""
    wl.cpu_step()                       # warm-up
    times = []
    t_begin = time.perf_counter()
    while len(times) < wl.cpu_repeats or (time.perf_counter() - t_begin < budget_s and len(times) < 3 * wl.cpu_repeats):
        t0 = time.perf_counter()
        wl.cpu_step()
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_begin > 3 * budget_s:
            break
    times.sort()
    return times[len(times) // 2], len(times)


def launch_floor_us(steps=200):
    """Microseconds per launch of a kernel that does nothing but one 4-byte store, replayed from a
    HIP graph like the microsecond workloads: what any kernel costs here before it moves a byte."""
    import torch
    from kraken_amd import _lib

    lib = _lib.load()
    word = torch.zeros(1, dtype=torch.int32, device="cuda")

    class _Floor:
        use_graph = True

        def step(self, i):
            lib.kr_stream_write_value32(word.data_ptr(), 1, torch.cuda.current_stream().cuda_stream)

    return time_gpu_graph(_Floor(), steps, 5)[1] * 1e3


def target_of(name, rec):
    """The benchmark definition's target for a workload and whether the measured figure meets it."""
    roof, frac = TARGETS.get(name, (None, None))
    if roof is None:
        return {"target": None, "meets_target": None}
    got = rec["mfma_frac"] if roof == "mfma" else rec["hbm_frac"]
    return {"target": {"roof": roof, "frac": frac}, "meets_target": bool(got >= frac)}


def measure(wl, steps, warmup, dev, with_cpu, cpu_budget):
    import torch

    wl.setup(dev)
    parity = wl.check()
    wall_ms, ev_ms = time_gpu(wl, steps, warmup)
    rec = {
        "workload": wl.name,
        "parity": parity,
        "ms_per_step": wall_ms,
        "kernel_ms": ev_ms,
        "gbps": wl.bytes / (ev_ms * 1e-3) / 1e9,
        "hbm_frac": wl.bytes / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "bound": wl.bound,
        "timing": "hip graph replay" if getattr(wl, "use_graph", False) else "eager launches",
        "algorithmic_bytes": wl.bytes,
        "traffic": MEASURED_TRAFFIC.get(wl.name),
        **wl.describe(),
    }
    if wl.flops:
        rec["tflops"] = wl.flops / (ev_ms * 1e-3) / 1e12
        rec["mfma_frac"] = rec["tflops"] / MFMA_BF16_PEAK_TFLOPS
        rec["algorithmic_flops"] = wl.flops
    rec.update(target_of(wl.name, rec))
    if with_cpu:
        cpu_s, n = time_cpu(wl, cpu_budget)
        rec["cpu_ms"] = cpu_s * 1e3
        rec["cpu_runs"] = n
        rec["cpu_gbps"] = wl.bytes / cpu_s / 1e9
        if wl.flops:
            rec["cpu_tflops"] = wl.flops / cpu_s / 1e12
    return rec


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2_one_shot", choices=sorted(make_workloads()))
    ap.add_argument("--all", dest="all", action="store_true", default=True,
                    help="also measure the other benchmark configurations (default)")
    ap.add_argument("--only", dest="all", action="store_false", help="measure only --workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="instead of a workload, run plain device copies of 256 MiB (a kernel of known "
                         "traffic: 268435456 B read + 268435456 B written per launch) to scale profiler counters")
    ap.add_argument("--sweep", default=None,
                    choices=["all_reduce", "all_reduce_bias", "all_reduce_bias_rms_norm", "matmul_reduce_scatter",
                             "all_gather_matmul"],
                    help="instead of the JSON line, sweep shapes and print a backend table like the reference's "
                         "benchmark/benchmark_*.py (first backend = baseline)")
    ap.add_argument("--backend", nargs="+", default=None, help="--sweep: backends to compare (default: all)")
    ap.add_argument("--shape", nargs="+", default=None,
                    help="--sweep: shapes, comma separated (e.g. 1024,6656,8192; a single number for all_reduce)")
    ap.add_argument("--world-size", type=int, default=8, help="--sweep: number of ranks whose buffers are reduced")
    ap.add_argument("--save-path", default=None, help="--sweep: also write the table as CSV")
    ap.add_argument("--plot-path", default=None, help="--sweep: also plot time against shape, one line per backend (PNG)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        _die_multi_gpu(max(args.gpus, int(os.environ.get("WORLD_SIZE", "1"))))

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible; this benchmark measures the GPU path only.", file=sys.stderr)
        sys.exit(3)
    import kraken_amd

    kraken_amd._lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    threads = torch.get_num_threads()

    if args.sweep:
        from kraken_amd._logging.sweep import run_sweep

        shapes = None
        if args.shape:
            shapes = [tuple(int(x) for x in sh.split(",")) for sh in args.shape]
            if args.sweep == "all_reduce":
                shapes = [sh[0] for sh in shapes]
        run_sweep(args.sweep, args.backend, shapes, args.world_size, args.save_path, dev=dev, plot_path=args.plot_path)
        return

    if args.calibrate_copy:
        src = torch.empty(128 * 1024 * 1024, dtype=torch.bfloat16, device=dev).normal_()
        dsts = [torch.empty_like(src) for _ in range(3)]
        for i in range(args.steps):
            dsts[i % 3].copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy": True, "launches": args.steps, "read_bytes": src.numel() * 2,
                          "write_bytes": src.numel() * 2}))
        return

    wls = make_workloads()
    main_wl = wls[args.workload]()
    rec = measure(main_wl, args.steps, args.warmup, dev, not args.no_cpu, 12.0)
    is_mfma = main_wl.bound == "mfma"
    value = rec["tflops"] if is_mfma else rec["gbps"]
    line = {
        "metric": "bf16 TFLOP/s, GEMM + reduce epilogue" if is_mfma else "HBM GB/s, W-way reduce (algorithmic bytes / time)",
        "value": value,
        "unit": "TFLOP/s" if is_mfma else "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": rec["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": main_wl.name, **main_wl.describe()},
        "parity": rec["parity"],
        "roofline": {
            "bound": main_wl.bound,
            "achieved": (rec["tflops"] if is_mfma else rec["gbps"]),
            "peak": MFMA_BF16_PEAK_TFLOPS if is_mfma else HBM_PEAK_GBS,
            "unit": "TFLOP/s" if is_mfma else "GB/s",
            "frac": (rec["mfma_frac"] if is_mfma else rec["hbm_frac"]),
            "traffic": MEASURED_TRAFFIC.get(main_wl.name),
            "kernel_ms": rec["kernel_ms"],
            "algorithmic_bytes": main_wl.bytes,
            "algorithmic_flops": main_wl.flops,
        },
        "target": rec["target"],
        "meets_target": rec["meets_target"],
    }
    if not args.no_cpu:
        line["cpu_baseline"] = {
            "value": rec["cpu_tflops"] if is_mfma else rec["cpu_gbps"],
            "unit": "TFLOP/s" if is_mfma else "GB/s",
            "cores": threads,
            "host_cpus": os.cpu_count(),
            "kind": "port",
            "sample": f"whole workload, median of {rec['cpu_runs']} runs of the oracle's torch-CPU math "
                      f"({rec['cpu_ms']:.1f} ms per pass)",
        }
    del main_wl
    torch.cuda.empty_cache()

    if args.all:
        others = []
        for key, ctor in wls.items():
            if key == args.workload:
                continue
            wl = ctor()
            big_gemm = wl.bound == "mfma" or wl.flops
            # GEMM steps take ~0.4 ms: half as many timed steps, but a longer warm-up -- the
            # matrix-core clocks need some tens of milliseconds of load to settle
            steps = max(10, args.steps // 2) if big_gemm else args.steps
            try:
                r = measure(wl, steps, max(args.warmup, 60) if big_gemm else args.warmup, dev, not args.no_cpu, 6.0)
                r["steps"] = steps
            except Exception as e:  # a failing side workload must not hide the headline number
                r = {"workload": wl.name, "error": f"{type(e).__name__}: {e}"}
            others.append(r)
            del wl
            torch.cuda.empty_cache()
        line["configs"] = others
        # what a launch costs before it moves a byte, in the protocol of the microsecond workloads
        # (the decode shape and the 256-row shape are reported beside it)
        line["launch_floor_us"] = launch_floor_us()
        met = [r.get("meets_target") for r in others] + [line["meets_target"]]
        line["targets_met"] = f"{sum(1 for m in met if m)} of {sum(1 for m in met if m is not None)} stated targets"
    print(json.dumps(line))


if __name__ == "__main__":
    main()
