"""CPU restatement (torch, fp32) of the arithmetic of Kraken's fused kernels.

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` may import this module; nothing under
``kraken_amd/`` does, and the product has no path that falls back to it.

The reference (``/root/reference``, Python + Triton + NVIDIA PTX) cannot run
without NVIDIA GPUs, NCCL and >= 4 ranks, and it holds no stored golden
vectors: its tests compute goldens live from ``dist.all_reduce``, ``torch.matmul``
and its own ``rms_norm`` and compare within 1e-2 .. 1e-1.  This oracle therefore
restates, function by function, the math those kernels and tests define, citing
the reference lines it follows.  What pins each function (see
``tests/test_oracle.py``):

* W-way sum / bias: an independent plain-C restatement (``oracle/oracle_c.c``)
  must agree bit for bit; closed forms (slices = (r+1)*c  =>  c*W(W+1)/2, adapted
  from ``test/test_gemm_allreduce.py:92-117``); W = 1 identity; brute force.
* RMSNorm: ``torch.nn.functional.rms_norm`` (library routine) must agree bit for
  bit on bf16; closed forms (constant row, zero row, unit weight => mean(y^2)=1,
  scale invariance).
* GEMM (+reduce / +band): the closed-form known-answer tests of the reference
  (``test/test_gemm_allreduce.py:92-117``, ``test/test_gemm_reduce_scatter.py:76-91``),
  identity-B, ones x ones = K, and a brute-force triple loop in C.
* fp8 branch of the all-gather matmul (``all_gather_matmul_fp8``): closed forms on
  exactly representable values, and a brute-force search of the nearest e4m3 value
  (ties to the even code) over the table of all 254 finite codes for products
  computed exactly in float64.  The reference holds no test of this branch and the
  saturating conversion is read off the instruction Triton emits for
  ``.to(tl.float8e4nv)`` on NVIDIA hardware: beyond its definition this function is
  "parity unpinned".

Beyond the tolerance bands of the reference's tests (1e-2 .. 1e-1) the
reference's bit-level behaviour (Triton ``tl.sum`` tree order, ``rsqrt.approx``,
TF32 ``tl.dot``, the bf16 accumulation of ``comm/one_shot_all_reduce.py:40-46``)
is "parity unpinned": nothing in this container can produce it.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

BF16 = torch.bfloat16


# --------------------------------------------------------------------------------------
# W-way reduce (+bias)
# --------------------------------------------------------------------------------------
def reduce(stack: torch.Tensor, bias: torch.Tensor | None = None, bias_first: bool = True) -> torch.Tensor:
    """``bf16([bias] + sum_r fp32(stack[r]))`` in ascending r, fp32, one rounding.

    one-shot order (bias first):  kraken/fused/one_shot_all_reduce_bias.py:80-93
    two-shot order (bias last):   kraken/fused/two_shot_all_reduce_bias.py:71-83
    no bias:                      kraken/comm/two_shot_all_reduce.py:56-62
    (kraken/comm/one_shot_all_reduce.py:40-46 accumulates in bf16 instead; the
    fp32 form is the one this build is specified to compute.)
    ``bias`` has the shape of a slice or is a vector over the last dimension.
    """
    W = stack.shape[0]
    if bias is not None and bias_first:
        acc = bias.float().expand(stack.shape[1:]).clone()
    else:
        acc = torch.zeros(stack.shape[1:], dtype=torch.float32)
    for r in range(W):
        acc += stack[r].float()
    if bias is not None and not bias_first:
        acc += bias.float().expand(stack.shape[1:])
    return acc.to(BF16)


def reduce_library(stack: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """Same quantity through library reductions — the torch math of the reference's
    own golden: ``dist.all_reduce(x)`` then ``x + bias`` (test/test_allreduce_bias.py:49-51),
    with the all-reduce taken as an fp32 sum over the stacked slices."""
    acc = stack.float().sum(0)
    if bias is not None:
        acc = acc + bias.float()
    return acc.to(BF16)


def striped_indices(numel: int, W: int, block: int, rank: int) -> torch.Tensor:
    """Flat indices rank ``rank`` owns under the two-shot striping:
    ``offsets = block_start + rank*BLOCK_SIZE + arange(BLOCK_SIZE)`` for block_start
    in steps of ``BLOCK_SIZE*W``, masked by ``offsets < numel``
    (kraken/comm/two_shot_all_reduce.py:51-55,146)."""
    idx = []
    start = 0
    while start < numel:
        lo = start + rank * block
        hi = min(lo + block, numel)
        if lo < hi:
            idx.append(torch.arange(lo, hi))
        start += block * W
    return torch.cat(idx) if idx else torch.zeros(0, dtype=torch.long)


def reduce_striped(stack: torch.Tensor, bias: torch.Tensor | None, block: int, rank: int) -> torch.Tensor:
    """This rank's striped share of the two-shot reduce, compact
    (kraken/fused/two_shot_all_reduce_bias.py:66-83)."""
    W = stack.shape[0]
    flat = stack.reshape(W, -1)
    idx = striped_indices(flat.shape[1], W, block, rank)
    b = None if bias is None else bias.reshape(-1)[idx]
    return reduce(flat[:, idx], b, bias_first=False)


def reduce_rotated(inp: torch.Tensor, W: int, rank: int, acc_bf16: bool = True) -> torch.Tensor:
    """``out = sum_i inp[band (i + rank + 1) % W]`` in that order; the reference keeps the
    running sum in the input dtype (kraken/fused/gemm_reduce_scatter_ce_persistent.py:258-279)."""
    M, N = inp.shape
    rows = M // W
    bands = inp.reshape(W, rows, N)
    cur = (rank + 1) % W
    if acc_bf16:
        acc = bands[cur].clone()
        for i in range(1, W):
            cur = (i + rank + 1) % W
            acc = (acc.float() + bands[cur].float()).to(BF16)
        return acc
    acc = bands[cur].float()
    for i in range(1, W):
        cur = (i + rank + 1) % W
        acc = acc + bands[cur].float()
    return acc.to(BF16)


# --------------------------------------------------------------------------------------
# RMSNorm
# --------------------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """kraken/fused/rms_norm.py:34-43: ``row`` in fp32, ``variance = sum(row*row)/D``,
    ``rstd = rsqrt(variance + eps)``, ``y = row * rstd * w`` rounded once at the store."""
    row = x.float()
    variance = (row * row).sum(-1, keepdim=True) / x.shape[-1]
    rstd = torch.rsqrt(variance + eps)
    return (row * rstd * w.float()).to(BF16)


def reduce_bias_rms_norm(stack: torch.Tensor, bias: torch.Tensor | None, w: torch.Tensor,
                         eps: float = 1e-5) -> torch.Tensor:
    """kraken/fused/one_shot_all_reduce_bias_rms_norm.py:73-91: ``row = fp32(bias)``;
    ``row += fp32(x_r)`` for r = 0..W-1; then the norm on the fp32 row."""
    W = stack.shape[0]
    if bias is not None:
        row = bias.float().expand(stack.shape[1:]).clone()
    else:
        row = torch.zeros(stack.shape[1:], dtype=torch.float32)
    for r in range(W):
        row += stack[r].float()
    variance = (row * row).sum(-1, keepdim=True) / stack.shape[-1]
    rstd = torch.rsqrt(variance + eps)
    return (row * rstd * w.float()).to(BF16)


def reduce_bias_rms_norm_library(stack: torch.Tensor, bias: torch.Tensor | None, w: torch.Tensor,
                                 eps: float = 1e-5) -> torch.Tensor:
    """The docstring form of the reference (one_shot_all_reduce_bias_rms_norm.py:112-116):
    ``dist.all_reduce(x); x = x + bias; y = F.rms_norm(x, x.shape[-1], w, eps)``, the
    all-reduce taken as an fp32 sum and the row kept in fp32 as the kernel does."""
    s = stack.float().sum(0)
    if bias is not None:
        s = s + bias.float()
    return F.rms_norm(s, (stack.shape[-1],), w.float(), eps).to(BF16)


# --------------------------------------------------------------------------------------
# GEMM + reduce
# --------------------------------------------------------------------------------------
def gemm_all_reduce(a: torch.Tensor, b: torch.Tensor, peers: torch.Tensor | None = None,
                    bias: torch.Tensor | None = None, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``a@b`` (fp32 accumulate) + the other ranks' partial products (+ bias):
    kraken/fused/gemm_one_shot_all_reduce_fused.py:56-64 (local product), :85-92 (sum over
    ranks), fp32 output :135; golden of the reference test: ``matmul`` then ``all_reduce``
    (test/test_gemm_allreduce.py:64-65)."""
    acc = a.float() @ b.float()
    if peers is not None:
        for j in range(peers.shape[0]):
            acc = acc + peers[j].float()
    if bias is not None:
        acc = acc + bias.float()
    return acc.to(out_dtype)


def gemm_reduce_scatter(a: torch.Tensor, b: torch.Tensor, peers: torch.Tensor | None, rank: int,
                        world_size: int, out_dtype: torch.dtype | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Full product, then this rank's ``M // world_size`` rows summed over ranks:
    kraken/fused/gemm_reduce_scatter_fused.py:63-69 (product), :102-114 (band), :118-127 (sum);
    golden of the reference test: ``reduce_scatter_tensor(matmul(a, b))``
    (test/test_gemm_reduce_scatter.py:102-108).  Returns (band result, full bf16 C)."""
    c = a.float() @ b.float()
    rows = a.shape[0] // world_size
    acc = c[rank * rows:(rank + 1) * rows].clone()
    if peers is not None:
        for j in range(peers.shape[0]):
            acc = acc + peers[j].float()
    return acc.to(out_dtype or a.dtype), c.to(BF16)


def all_gather_matmul(a_stack: torch.Tensor, b: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``A = concat_r a_stack[r]`` (exact copy, test/test_allgather_matmul.py:75) and
    ``C = A @ b`` in bf16 with fp32 accumulation (kraken/fused/all_gather_matmul.py:115-123)."""
    W, m, K = a_stack.shape
    a_full = a_stack.reshape(W * m, K)
    return a_full, (a_full.float() @ b.float()).to(a_stack.dtype)


# --------------------------------------------------------------------------------------
# Deterministic synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------------------
def all_gather_matmul_fp8(a_stack: torch.Tensor, b: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The fp8 branch of the all-gather matmul (kraken/fused/all_gather_matmul.py:53,121,213): fp8
    (e4m3fn) operands, fp32 accumulate, the result rounded to fp8 once.  The rounding is torch's
    (nearest even), clamped to +-448 first: the reference's generated conversion saturates where
    torch's gives NaN, from magnitude 464 on."""
    W, m, K = a_stack.shape
    a_full = a_stack.reshape(W * m, K)
    c = torch.matmul(a_full.float(), b.float()).clamp(-448.0, 448.0)
    return a_full, c.to(torch.float8_e4m3fn)


def randn_bf16(shape, seed: int, std: float = 1.0, mean: float = 0.0) -> torch.Tensor:
    """fp32 normal draw from a seeded CPU generator, scaled, cast to bf16."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std + mean).to(BF16)


def make_stack(W: int, shape, seed0: int = 42) -> torch.Tensor:
    """Slice r is drawn with seed ``seed0 + r`` (mirrors ``torch.manual_seed(42 + rank)``,
    test/test_allreduce.py:46)."""
    return torch.stack([randn_bf16(shape, seed0 + r) for r in range(W)])


def make_bias_weight(D: int, seed: int = 42) -> tuple[torch.Tensor, torch.Tensor]:
    """bias ~ N(0, 0.02), weight ~ 1 + N(0, 0.02), both bf16 [D]."""
    return randn_bf16((D,), seed, 0.02), randn_bf16((D,), seed + 1000, 0.02, 1.0)
