#!/usr/bin/env python3
"""Benchmark of the one-rank hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all]

A "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM.  The default workload is the configuration the
headline metric is quoted on: the pure one-shot W-way reduce, bf16
[8,4096,4096] -> [4096,4096] (HBM-bound).  One JSON line is printed; with
``--all`` (default) the line also carries, under "configs", the other
benchmark configurations (reduce+bias+RMSNorm, two-shot share, decode shape,
GEMM + reduce-scatter, GEMM + fused all-reduce, all-gather matmul, and the
copy-engine reduce-scatter and overlapped all-gather matmul at the reference's
test shapes), each checked against the CPU oracle before it is timed.

Timing (the method of the reference's benchmark_with_event,
kraken/_logging/benchmarking.py:91-163: warm-up, one event interval per
iteration, median): W untimed warm-up steps, then the same workload for a
fixed time (SETTLE_MS of launches, so that clocks and power state do not
depend on what ran before), then exactly K steps between two device
synchronisations with an event recorded on the launch stream before each
interval and after the last (an interval is one step for the GEMMs and as many
steps as last 0.25 ms for shorter kernels, since an event between two launches
costs about 2 us that would be charged to the kernel); the median of the
intervals is the kernel time the roofline figure uses, minimum and maximum are
reported beside it.
Workloads of a few microseconds are replayed from a HIP graph of G launches
instead (the host cannot enqueue them as fast as the GPU retires them): R
replays, each between its own pair of events, median of replay / G.  Every
workload rotates several complete operand sets (inputs, peers and outputs,
the GEMM operands A and B included), together larger than the 256 MB
last-level cache, so no step finds its operands cached.  All GPU timings
come first; the CPU baseline legs (the oracle's torch-CPU math on the same
inputs) run after the last of them.  Each entry states the target the
benchmark definition gives for it (a fraction of the HBM or bf16 matrix-core
peak) and whether the measured figure meets it; the GEMM entries carry the
vendor library's time for the bare product of the same operands, measured the
same way in the same run, and the microsecond entries the cost of a launch
that does nothing, of one that only reads the input and of a plain copy of
the same number of bytes.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
MFMA_FP8_PEAK_TFLOPS = 5000.0    # MI355X dense fp8
W = 8
SETTLE_MS = 60.0                 # launches of the workload itself in front of every timed region
GRAPH_REPLAYS = 15               # timed replays of a microsecond workload's graph
MIN_EAGER_STEPS = 30             # timed launches of a side workload that is not replayed from a graph

# HBM-side bytes per launch of the dominant kernel (L2 fills + write-backs), from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of `bench.py --only --no-cpu --workload <key>`, each counter scaled by
# what it reads for a plain 256 MiB device copy (`bench.py --calibrate-copy`).  bench.py cannot read
# hardware counters itself; the figures and the commands behind them are kept as text under
# profiles/ (one file per kernel and workload).  Each entry: (bytes, commit of the kernel source the
# profile was taken at); the JSON carries both, so a figure that predates a kernel change shows.
MEASURED_TRAFFIC = {
    "one_shot_reduce_w8_4096x4096": (302051604, "8eb5098"),             # profiles/reduce_kernel_w8_4096x4096.md
    "two_shot_share_w8_512x4096": (37836204, "8eb5098"),                # profiles/reduce_kernel_w8_two_shot_share_512x4096.md
    "reduce_bias_rmsnorm_w8_256x4096": (19048668, "8eb5098"),           # profiles/reduce_rmsnorm_kernel_w8_256x4096.md
    "reduce_bias_rmsnorm_w8_16x8192_decode": (2494411, "8eb5098"),      # profiles/reduce_rmsnorm_split_kernel_w8_16x8192.md
    "reduce_bias_rmsnorm_w8_16384x4096_large": (1208007579, "8eb5098"), # profiles/reduce_rmsnorm_kernel_w8_16384x4096.md
    # the GEMMs: L2 fills (A and B panels re-read per tile row / column, served mostly by the 256 MB
    # last-level cache, not by HBM) + write-backs
    "gemm_reduce_scatter_8192x8192x3584_w8": (986499754, "ffe923e"),    # profiles/gemm_dtl16_kernel_reduce_scatter_8192x8192x3584.md
    "gemm_all_reduce_4096x8192x1024_w8": (708047563, "ffe923e"),        # profiles/gemm_dtl16_kernel_all_reduce_4096x8192x1024.md
    "all_gather_matmul_8192x3584x8192_w8": (837421610, "ffe923e"),      # profiles/gemm_dtl16n7_kernel_all_gather_matmul_8192x3584x8192.md
    "all_gather_matmul_4096x6656x16384_w8": (1894179528, "ffe923e"),    # profiles/gemm_dtl16_kernel_all_gather_matmul_4096x6656x16384.md
    "all_gather_matmul_fp8_4096x6656x16384_w8": (851641889, "ffe923e"),  # profiles/gemm_dtl8_kernel_all_gather_matmul_fp8_4096x6656x16384.md
}

# Targets of the benchmark definition: fraction of the binding roof.  The W = 8 reduce(+bias+RMSNorm)
# paths: 75 % of peak HBM bandwidth; the GEMM + reduce paths at the Llama-70B TP8 shard shapes: 60 %
# of the dense bf16 matrix-core peak.  The decode shape is latency-bound (reported in microseconds
# beside the launch floor) and the fused GEMM + all-reduce is HBM-bound (122 flop/B: its matrix-core
# fraction cannot exceed 39 %), so neither has a target of its own; the two shapes taken from the
# reference's tests are reported without one.
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
    use_graph = False      # microsecond kernels: time replays of a HIP graph of the launches
    has_vendor = False     # GEMMs: vendor_step() runs the vendor library's bare product
    vendor_what = "torch.matmul (hipBLASLt) of the same A and B, product only"
    mfma_peak = MFMA_BF16_PEAK_TFLOPS   # matrix-core peak of the workload's arithmetic type

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

    def release(self):
        """Drop every device tensor (the host inputs stay for the CPU leg)."""
        import torch

        def on_device(v):
            if isinstance(v, torch.Tensor):
                return v.is_cuda
            if isinstance(v, (list, tuple)):
                return any(on_device(x) for x in v)
            return False

        for k in [k for k, v in vars(self).items() if on_device(v)]:
            delattr(self, k)


def _rand_sets(shape, nsets, dev, std=1.0, seed=1234):
    import torch

    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    return [(torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * std).to(torch.bfloat16)
            for _ in range(nsets)]


def _flat_bytes(t):
    import torch

    return t.reshape(-1).view(torch.uint8)


class OneShotReduce(Workload):
    """benchmark config 2: stack [8,4096,4096] -> [4096,4096]."""
    name = "one_shot_reduce_w8_4096x4096"
    R, D = 4096, 4096
    nsets = 4   # 4 x 256 MiB of input: no step finds its input in the 256 MB last-level cache

    def __init__(self):
        self.bytes = (W + 1) * self.R * self.D * 2

    def setup(self, dev):
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

    def describe(self):
        return {"W": W, "shape": [W, self.R // W, self.D], "of_stack": [W, self.R, self.D],
                "out": [self.R // W, self.D], "kernel": "reduce_kernel"}

    def floor_src(self, i):
        # as many contiguous input bytes as a share reads (8 x 4 MiB), a different region every launch
        n = W * (self.R // W) * self.D * 2
        flat = _flat_bytes(self.sets[i % self.nsets])
        r = (i // self.nsets) % (flat.numel() // n)
        return flat[r * n:(r + 1) * n]


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

    def floor_src(self, i):
        return _flat_bytes(self.sets[i % self.nsets])


def _vendor_matmul(a, b, out):
    import torch

    torch.matmul(a, b, out=out)


class GemmReduceScatter(Workload):
    """benchmark config 4: A [8192,3584] @ B [3584,8192]; own 1024-row band + 7 partials."""
    name = "gemm_reduce_scatter_8192x8192x3584_w8"
    bound = "mfma"
    M, N, K = 8192, 8192, 3584
    cpu_repeats = 3
    nsets = 3   # 3 x 369 MB of A, B, peers and outputs in rotation: every step's operands come from HBM
    has_vendor = True

    def __init__(self):
        self.flops = 2 * self.M * self.N * self.K
        # A + B + every row of C written once (the band's rows to `out`, the others to the C scratch)
        # + the 7 partials of the band
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

    def vendor_step(self, i):
        j = i % self.nsets
        _vendor_matmul(self.a[j], self.b[j], self.c[j])

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
        from kraken_amd import _lib

        plan = _lib.gemm_plan(self.M, self.N, self.K, False, W - 1, self.M // W, False, True)
        return {"M": self.M, "N": self.N, "K": self.K, "peers": [7, 1024, self.N], "b_layout": "row-major",
                "kernel": plan["kernel"], "plan": plan, "operand_sets": self.nsets}


class GemmAllReduce(Workload):
    """benchmark config 5 (fused): A [4096,1024] @ B [1024,8192] + 7 partials + bias; HBM-bound."""
    name = "gemm_all_reduce_4096x8192x1024_w8"
    bound = "hbm"
    M, N, K = 4096, 8192, 1024
    cpu_repeats = 3
    nsets = 2
    has_vendor = True

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
        self.vout = [torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev) for _ in range(self.nsets)]
        self.out = None

    def step(self, i):
        import torch
        from kraken_amd import fused

        j = i % self.nsets
        self.out = fused.gemm_one_shot_all_reduce_fused(self.a[j], self.b[j], peers=self.psets[j],
                                                        bias=self.bias, out_dtype=torch.bfloat16)

    def vendor_step(self, i):
        j = i % self.nsets
        _vendor_matmul(self.a[j], self.b[j], self.vout[j])

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
        from kraken_amd import _lib

        plan = _lib.gemm_plan(self.M, self.N, self.K, False, W - 1, self.M, True, False)
        return {"M": self.M, "N": self.N, "K": self.K, "peers": [7, self.M, self.N], "bias": [self.N],
                "b_layout": "row-major", "kernel": plan["kernel"], "plan": plan, "operand_sets": self.nsets}


class AllGatherMatmul(Workload):
    """All-gather matmul: A stack [W, m, K] @ B [K, N], B.T contiguous.

    Default shape: benchmark config 5 (all-gather), [8,1024,8192] @ [8192,3584].  ``gather=True``
    is the reference's overlapped form: the shards are copied into the gathered matrix chunk by
    chunk on a side stream while the GEMM's tiles wait for their chunk's flag."""
    bound = "mfma"
    cpu_repeats = 3
    has_vendor = True

    def __init__(self, m=1024, K=8192, N=3584, nsets=3, gather=False):
        self.m, self.K, self.N, self.nsets, self.gather = m, K, N, nsets, gather
        self.name = f"all_gather_matmul_{W * m}x{N}x{K}_w8" + ("_overlapped" if gather else "")
        self.flops = 2 * W * m * N * K
        self.bytes = (W * m * K + K * N + W * m * N) * 2
        if gather:   # the shards are read and the gathered matrix is written once more
            self.bytes += 2 * W * m * K * 2

    def setup(self, dev):
        import torch
        from oracle import oracle as orc

        self.hs = orc.make_stack(W, (self.m, self.K), seed0=42)
        self.hbT = orc.randn_bf16((self.N, self.K), 43, 0.02)
        self.s = [self.hs.to(dev)] + _rand_sets((W, self.m, self.K), self.nsets - 1, dev, seed=1)
        self.bT = [self.hbT.to(dev)] + _rand_sets((self.N, self.K), self.nsets - 1, dev, std=0.02, seed=2)
        self.c = [None] * self.nsets
        self.vout = [torch.empty(W * self.m, self.N, dtype=torch.bfloat16, device=dev) for _ in range(self.nsets)]
        if self.gather:
            self.a_out = [torch.empty(W * self.m, self.K, dtype=torch.bfloat16, device=dev) for _ in range(self.nsets)]
            self.progress = torch.zeros(W, dtype=torch.int32, device=dev)

    def step(self, i):
        from kraken_amd import fused

        j = i % self.nsets
        self.c[j] = None                         # (the allocator hands this set's own block back)
        if self.gather:
            _, self.c[j] = fused.all_gather_matmul(self.s[j], self.bT[j].T, self.a_out[j], self.progress, rank=3,
                                                   gather=True)
        else:
            _, self.c[j] = fused.all_gather_matmul(self.s[j], self.bT[j].T, rank=3)

    def vendor_step(self, i):
        j = i % self.nsets
        _vendor_matmul(self.s[j].reshape(-1, self.K), self.bT[j].T, self.vout[j])

    def check(self):
        import torch

        self.step(0)
        rows = W * self.m
        pick = torch.tensor([0, self.m - 1, 3 * self.m, rows - 1])
        want = self.hs.reshape(-1, self.K)[pick].float() @ self.hbT.T.float()
        torch.testing.assert_close(self.c[0].cpu()[pick].float(), want.to(torch.bfloat16).float(), rtol=2e-2, atol=2e-2)
        if self.gather:
            from kraken_amd import _waits

            _waits.check(block=True)
            assert torch.equal(self.a_out[0].cpu()[pick], self.hs.reshape(-1, self.K)[pick]), "gathered A differs"
            return "sampled rows within rtol=atol=2e-2 of the oracle, gathered rows bit-exact"
        return "sampled rows within rtol=atol=2e-2 of the oracle"

    def cpu_step(self):
        from oracle import oracle as orc

        return orc.all_gather_matmul(self.hs, self.hbT.T)

    def describe(self):
        from kraken_amd import _lib

        plan = _lib.gemm_plan(W * self.m, self.N, self.K, True,
                              workspace_bytes=_lib.load().kr_gemm_workspace_bytes(W * self.m, self.N, self.K))
        d = {"W": W, "m": self.m, "K": self.K, "N": self.N, "b_layout": "b.T contiguous", "kernel": plan["kernel"],
             "plan": plan, "operand_sets": self.nsets}
        if self.gather:
            d["overlap"] = "8 shard copies + flag writes on a side stream while the tiles wait for their shard"
        return d


class AllGatherMatmulFP8(AllGatherMatmul):
    """The fp8 branch of the all-gather matmul (kraken/fused/all_gather_matmul.py:53,121,213) at the
    reference's test shape: fp8 (e4m3fn) shards and weight, fp32 accumulation on the fp8 matrix-core
    instruction, fp8 result.  Priced against the fp8 peak."""
    dtype = "fp8 (e4m3fn) storage, fp32 accumulate"
    mfma_peak = MFMA_FP8_PEAK_TFLOPS
    vendor_what = "torch._scaled_mm (hipBLASLt) of the same fp8 A and B with unit scales, bf16 result"

    def __init__(self, m=512, K=16384, N=6656, nsets=2):
        super().__init__(m, K, N, nsets, False)
        self.name = f"all_gather_matmul_fp8_{W * m}x{N}x{K}_w8"
        self.bytes = W * m * K + K * N + W * m * N

    def setup(self, dev):
        import torch

        fp8 = torch.float8_e4m3fn
        g = torch.Generator().manual_seed(44)
        self.hs = torch.randn(W, self.m, self.K, generator=g).to(fp8)
        self.hbT = (torch.randn(self.N, self.K, generator=g) * 0.02).to(fp8)
        gd = torch.Generator(device=dev).manual_seed(3)
        self.s = [self.hs.to(dev)] + [torch.randn(W, self.m, self.K, generator=gd, device=dev).to(fp8) for _ in range(self.nsets - 1)]
        self.bT = [self.hbT.to(dev)] + [(torch.randn(self.N, self.K, generator=gd, device=dev) * 0.02).to(fp8)
                                        for _ in range(self.nsets - 1)]
        self.c = [None] * self.nsets
        self.one = torch.ones((), device=dev)

    def vendor_step(self, i):
        import torch

        j = i % self.nsets
        torch._scaled_mm(self.s[j].reshape(-1, self.K), self.bT[j].T, scale_a=self.one, scale_b=self.one, out_dtype=torch.bfloat16)

    def check(self):
        import torch
        from oracle import oracle as orc

        self.step(0)
        rows = W * self.m
        pick = torch.tensor([0, self.m - 1, 3 * self.m, rows - 1])
        _, want = orc.all_gather_matmul_fp8(self.hs.reshape(-1, self.K)[pick].reshape(1, len(pick), self.K), self.hbT.T)
        got, ref = self.c[0].cpu()[pick].float(), want.float()
        step = torch.maximum(ref.abs(), torch.tensor(2.0 ** -6)) * 2.0 ** -3      # spacing of e4m3 at that magnitude
        assert ((got - ref).abs() <= step).all() and (got == ref).float().mean() > 0.98, "fp8 result differs from the oracle"
        return "sampled rows within one fp8 step of the oracle (the orders of the fp32 sums differ), over 98 % equal"

    def cpu_step(self):
        from oracle import oracle as orc

        return orc.all_gather_matmul_fp8(self.hs, self.hbT.T)

    def describe(self):
        return {"W": W, "m": self.m, "K": self.K, "N": self.N, "b_layout": "b.T contiguous", "kernel": "gemm_dtl8_kernel",
                "operand_sets": self.nsets, "mfma": "v_mfma_f32_16x16x128_f8f6f4", "peak_priced_against": "fp8 dense, 5.0 PFLOP/s"}


class GemmReduceScatterCE(Workload):
    """Copy-engine reduce-scatter variant at the reference's test shape
    (test/test_gemm_reduce_scatter.py:93-111): producer GEMM with per-band flags, band copies,
    rotated-order band reduce."""
    name = "gemm_reduce_scatter_ce_persistent_8192x4096x14336_w8"
    bound = "mfma"
    M, N, K = 8192, 4096, 14336
    cpu_repeats = 3
    nsets = 2
    has_vendor = True

    def __init__(self):
        self.flops = 2 * self.M * self.N * self.K
        band = (self.M // W) * self.N
        # A, B, C written; the own band and the 7 arriving bands copied into the scatter buffer (read +
        # write each); the W bands read by the reduce, one band written
        self.bytes = (self.M * self.K + self.K * self.N + self.M * self.N + 2 * W * band + W * band + band) * 2

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
        self.vout = [torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev) for _ in range(self.nsets)]
        self.out = None

    def step(self, i):
        from kraken_amd import fused

        j = i % self.nsets
        self.out = fused.gemm_reduce_scatter_ce_persistent(self.a[j], self.b[j], peers=self.p[j], rank=self.rank)

    def vendor_step(self, i):
        j = i % self.nsets
        _vendor_matmul(self.a[j], self.b[j], self.vout[j])

    def check(self):
        import torch

        self.step(0)
        r0 = self.rank * (self.M // W)
        pick = torch.tensor([0, 255, 256, self.M // W - 1])
        own = (self.ha[r0 + pick].float() @ self.hb.float()).to(torch.bfloat16).float()
        want = own + self.hp[:, pick].float().sum(0)
        # the reference's tolerance for this function (test/test_gemm_reduce_scatter.py:110): the running
        # sum is rounded to bf16 after every add, in rotated order
        torch.testing.assert_close(self.out.cpu()[pick].float(), want, rtol=2e-2, atol=1e-1)
        return "sampled rows within rtol=2e-2, atol=1e-1 of the fp32-accumulated oracle (the path rounds to bf16 after every add)"

    def cpu_step(self):
        from oracle import oracle as orc

        return orc.gemm_reduce_scatter(self.ha, self.hb, self.hp, self.rank, W)

    def describe(self):
        from kraken_amd import _lib

        plan = _lib.gemm_plan(self.M, self.N, self.K, False)
        return {"M": self.M, "N": self.N, "K": self.K, "peers": [7, self.M // W, self.N], "b_layout": "row-major",
                "kernel": plan["kernel"], "plan": plan, "operand_sets": self.nsets,
                "launches": "producer GEMM (flags per band), band copies, reduce_rotated_kernel"}


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
        # the reference's own test shapes of the two overlap paths
        "ref_gemm_reduce_scatter_ce_persistent": GemmReduceScatterCE,
        "ref_all_gather_matmul": lambda: AllGatherMatmul(512, 16384, 6656, 2, False),
        "ref_all_gather_matmul_overlapped": lambda: AllGatherMatmul(512, 16384, 6656, 2, True),
        "ref_all_gather_matmul_fp8": AllGatherMatmulFP8,
    }


# --------------------------------------------------------------------------------------
# measurement
# --------------------------------------------------------------------------------------
def _stats(per_ms):
    return {"median_ms": statistics.median(per_ms), "min_ms": min(per_ms), "max_ms": max(per_ms), "n": len(per_ms)}


def _settle(run, min_ms):
    """Keep the GPU busy with `run()` (which enqueues a batch of the workload's launches) for at
    least `min_ms`: clocks and power state then belong to this workload and not to whatever ran,
    or idled, before it."""
    import torch

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n = 0
    while (time.perf_counter() - t0) * 1e3 < min_ms:
        run(n)
        torch.cuda.synchronize()
        n += 1
    return n


def time_gpu_graph(step, steps, warmup, nsets=1, replays=GRAPH_REPLAYS, settle_ms=SETTLE_MS):
    """Device time per launch with the launches replayed from one HIP graph.

    For workloads whose kernel runs only a few microseconds the host cannot enqueue launches
    as fast as the GPU retires them, and events around an eager loop would measure the host.
    (The reference's benchmark_with_event has the same option, _logging/benchmarking.py:98-108.)
    The graph holds G launches (at least `steps`, at least 96, a multiple of the number of operand
    sets so that consecutive replays keep rotating); `replays` replays are timed, each between its
    own pair of events, after the same graph has run untimed for `settle_ms`.  Returns
    (wall ms per launch over all timed replays, statistics of replay / G, launches timed).
    """
    import torch

    G = max(steps, 96)
    G = -(-G // nsets) * nsets
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step(0)
        with torch.cuda.graph(graph, stream=side):
            for i in range(G):
                step(warmup + i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    _settle(lambda n: [graph.replay() for _ in range(8)], settle_ms)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(replays)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(replays)]
    graph.replay()                       # one more untimed replay directly in front of the timed ones
    t0 = time.perf_counter()
    for r in range(replays):
        starts[r].record()
        graph.replay()
        ends[r].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    per = [s.elapsed_time(e) / G for s, e in zip(starts, ends)]
    return (t1 - t0) * 1e3 / (replays * G), _stats(per), replays * G


MIN_INTERVAL_MS = 0.25           # an event interval of the eager protocol covers at least this much GPU time


def time_gpu_eager(step, steps, warmup, settle_ms=SETTLE_MS):
    """Exactly `steps` launches between two synchronisations, with events on the launch stream
    that cut them into intervals: (wall ms per step, statistics of interval / its launches, steps).

    An event between two launches costs about 2 us of GPU time on this machine (the launches no
    longer run back to back), which would be charged to the kernel: an interval therefore covers
    as many launches as it takes to last MIN_INTERVAL_MS, and at least two -- two for the GEMMs,
    five for a 50 us kernel -- so that the markers stay below one percent of what they bracket.
    """
    import torch

    for i in range(warmup):
        step(i)
    _settle(lambda n: [step(warmup + k) for k in range(10)], settle_ms)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for k in range(10):
        step(warmup + k)
    b.record()
    torch.cuda.synchronize()
    est_ms = a.elapsed_time(b) / 10
    stride = max(2 if steps >= 8 else 1, min(steps, int(-(-MIN_INTERVAL_MS // est_ms))))
    n_int = -(-steps // stride)                               # intervals of equal length (to within one launch)
    marks = [j * steps // n_int for j in range(n_int)] + [steps]   # an event in front of these steps, and one at the end
    evs = [torch.cuda.Event(enable_timing=True) for _ in marks]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    nxt = 0
    for i in range(steps):
        if i == marks[nxt]:
            evs[nxt].record()            # on the current stream = the stream the kernels go to
            nxt += 1
        step(warmup + i)
    evs[nxt].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    per = [evs[j].elapsed_time(evs[j + 1]) / (marks[j + 1] - marks[j]) for j in range(len(marks) - 1)]
    st = _stats(per)
    st["launches_per_interval"] = steps // n_int
    return (t1 - t0) * 1e3 / steps, st, steps


def time_gpu(wl, steps, warmup):
    """(wall ms per step, interval statistics, steps really timed) for a workload."""
    if wl.use_graph:
        return time_gpu_graph(wl.step, steps, warmup, wl.nsets)
    return time_gpu_eager(wl.step, steps, warmup)


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

    def step(i):
        lib.kr_stream_write_value32(word.data_ptr(), 1, torch.cuda.current_stream().cuda_stream)

    _, st, _ = time_gpu_graph(step, steps, 5, settle_ms=20.0)
    return {k.replace("_ms", "_us"): (v * 1e3 if k != "n" else v) for k, v in st.items()}


def floors_of(wl, steps, warmup):
    """What the machine charges for launches of this workload's size that do no arithmetic, under
    the same replay protocol and on the same rotating inputs: a kernel that only reads the input
    (nothing written), and a plain copy that moves the workload's algorithmic bytes (half read,
    half written).  Microseconds per launch, median (min .. max)."""
    import torch
    from kraken_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda")
    in_bytes = wl.floor_src(0).numel()
    half = (wl.bytes // 2) // 16 * 16
    dsts = [torch.empty(half, dtype=torch.uint8, device=dev) for _ in range(4)]

    def read_step(i):
        src = wl.floor_src(i)
        rc = lib.kr_probe_read(src.data_ptr(), src.numel(), None, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc

    def copy_step(i):
        src = wl.floor_src(i)
        rc = lib.kr_probe_copy(src.data_ptr(), dsts[i % 4].data_ptr(), half, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc

    out = {}
    for key, fn, nbytes in (("read_input", read_step, in_bytes), ("copy_same_bytes", copy_step, 2 * half)):
        _, st, _ = time_gpu_graph(fn, steps, warmup, wl.nsets, settle_ms=20.0)
        out[key] = {"us": st["median_ms"] * 1e3, "min_us": st["min_ms"] * 1e3, "max_us": st["max_ms"] * 1e3,
                    "bytes": nbytes}
    return out


def target_of(name, rec):
    """The benchmark definition's target for a workload and whether the measured figure meets it."""
    roof, frac = TARGETS.get(name, (None, None))
    if roof is None:
        return {"target": None, "meets_target": None}
    got = rec["mfma_frac"] if roof == "mfma" else rec["hbm_frac"]
    return {"target": {"roof": roof, "frac": frac}, "meets_target": bool(got >= frac)}


def measure_gpu(wl, steps, warmup, dev, floors=False):
    """Set the workload up, check it against the oracle, time it (and the vendor product / the
    floors beside it), then drop its device tensors.  The CPU leg comes later (measure_cpu)."""
    wl.setup(dev)
    parity = wl.check()
    wall_ms, st, timed = time_gpu(wl, steps, warmup)
    ev_ms = st["median_ms"]
    traffic = MEASURED_TRAFFIC.get(wl.name, (None, None))
    rec = {
        "workload": wl.name,
        "parity": parity,
        "ms_per_step": wall_ms,
        "kernel_ms": ev_ms,
        "kernel_ms_min": st["min_ms"],
        "kernel_ms_max": st["max_ms"],
        "intervals": st["n"],
        "steps": timed,
        "gbps": wl.bytes / (ev_ms * 1e-3) / 1e9,
        "hbm_frac": wl.bytes / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "bound": wl.bound,
        "dtype": wl.dtype,
        "timing": (f"hip graph of {timed // st['n']} launches, median of {st['n']} replays" if wl.use_graph
                   else f"eager launches, median of {st['n']} event intervals of {st['launches_per_interval']} launch(es)"),
        "algorithmic_bytes": wl.bytes,
        "traffic": traffic[0],
        "traffic_profiled_at": traffic[1],
        **wl.describe(),
    }
    if wl.flops:
        rec["tflops"] = wl.flops / (ev_ms * 1e-3) / 1e12
        rec["mfma_frac"] = rec["tflops"] / wl.mfma_peak
        rec["algorithmic_flops"] = wl.flops
    is_mfma = wl.bound == "mfma"
    rec["roofline"] = {
        "bound": wl.bound,
        "achieved": rec["tflops"] if is_mfma else rec["gbps"],
        "peak": wl.mfma_peak if is_mfma else HBM_PEAK_GBS,
        "unit": "TFLOP/s" if is_mfma else "GB/s",
        "frac": rec["mfma_frac"] if is_mfma else rec["hbm_frac"],
        "traffic": traffic[0],
    }
    rec.update(target_of(wl.name, rec))
    if wl.has_vendor:
        # the vendor library's bare product of the same rotating operands (no peers, bias or band),
        # same protocol, same run
        _, vst, _ = time_gpu_eager(wl.vendor_step, max(steps, MIN_EAGER_STEPS), warmup)
        rec["vendor"] = {"what": wl.vendor_what,
                         "ms": vst["median_ms"], "min_ms": vst["min_ms"], "max_ms": vst["max_ms"],
                         "tflops": wl.flops / (vst["median_ms"] * 1e-3) / 1e12,
                         "mfma_frac": wl.flops / (vst["median_ms"] * 1e-3) / 1e12 / wl.mfma_peak}
    if floors and wl.use_graph and hasattr(wl, "floor_src"):
        rec["floors_us"] = floors_of(wl, steps, warmup)
    wl.release()
    return rec


def measure_cpu(wl, rec, budget_s):
    cpu_s, n = time_cpu(wl, budget_s)
    rec["cpu_ms"] = cpu_s * 1e3
    rec["cpu_runs"] = n
    rec["cpu_gbps"] = wl.bytes / cpu_s / 1e9
    if wl.flops:
        rec["cpu_tflops"] = wl.flops / cpu_s / 1e12


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
    ap.add_argument("--floors", action="store_true",
                    help="with --only: also time the launch, read-only and copy floors beside the workload "
                         "(always done for the microsecond workloads of the default run)")
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
    # ---- GPU legs: the headline workload first, then the others ---------------------------------
    rec = measure_gpu(main_wl, args.steps, args.warmup, dev, floors=args.floors or args.all)
    torch.cuda.empty_cache()
    others = []
    if args.all:
        for key, ctor in wls.items():
            if key == args.workload:
                continue
            wl = ctor()
            # side workloads that are not graph replays get at least MIN_EAGER_STEPS timed launches
            # (one event interval each)
            steps = args.steps if wl.use_graph else max(args.steps, MIN_EAGER_STEPS)
            try:
                r = measure_gpu(wl, steps, args.warmup, dev, floors=True)
            except Exception as e:  # a failing side workload must not hide the headline number
                r = {"workload": wl.name, "error": f"{type(e).__name__}: {e}"}
                wl.release()
            others.append((wl, r))
            torch.cuda.empty_cache()
        # what a launch costs before it moves a byte, in the protocol of the microsecond workloads
        floor = launch_floor_us()
    # ---- CPU legs, behind every GPU timing -------------------------------------------------------
    if not args.no_cpu:
        measure_cpu(main_wl, rec, 12.0)
        for wl, r in others:
            if "error" not in r:
                try:
                    measure_cpu(wl, r, 6.0)
                except Exception as e:
                    r["cpu_error"] = f"{type(e).__name__}: {e}"

    is_mfma = main_wl.bound == "mfma"
    value = rec["tflops"] if is_mfma else rec["gbps"]
    line = {
        "metric": (("fp8" if main_wl.mfma_peak == MFMA_FP8_PEAK_TFLOPS else "bf16") + " TFLOP/s, GEMM + reduce epilogue") if is_mfma
                  else "HBM GB/s, W-way reduce (algorithmic bytes / time)",
        "value": value,
        "unit": "TFLOP/s" if is_mfma else "GB/s",
        "n_gpus": 1,
        "steps": rec["steps"],
        "warmup": args.warmup,
        "settle_ms": SETTLE_MS,
        "ms_per_step": rec["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8" if is_mfma and main_wl.mfma_peak == MFMA_FP8_PEAK_TFLOPS else "bf16",
        "data": "synthetic",
        "config": {"workload": main_wl.name, **main_wl.describe()},
        "parity": rec["parity"],
        "timing": rec["timing"],
        "roofline": {
            **rec["roofline"],
            "kernel_ms": rec["kernel_ms"],
            "kernel_ms_min": rec["kernel_ms_min"],
            "kernel_ms_max": rec["kernel_ms_max"],
            "traffic_profiled_at": rec["traffic_profiled_at"],
            "algorithmic_bytes": main_wl.bytes,
            "algorithmic_flops": main_wl.flops,
        },
        "target": rec["target"],
        "meets_target": rec["meets_target"],
    }
    for k in ("vendor", "floors_us"):
        if k in rec:
            line[k] = rec[k]
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
    if args.all:
        line["configs"] = [r for _, r in others]
        line["launch_floor_us"] = floor["median_us"]
        line["launch_floor"] = floor
        for r in line["configs"]:
            if "floors_us" in r:
                r["floors_us"]["launch"] = {"us": floor["median_us"], "min_us": floor["min_us"], "max_us": floor["max_us"]}
        met = [r.get("meets_target") for r in line["configs"]] + [line["meets_target"]]
        line["targets_met"] = f"{sum(1 for m in met if m)} of {sum(1 for m in met if m is not None)} stated targets"
    print(json.dumps(line))


if __name__ == "__main__":
    main()
