"""Seeded random shapes through every kernel family, each checked against the CPU oracle at the
gate of its family: reduce (+bias) bit-exact; reduce+bias+RMSNorm within one bf16 ulp and
rtol = atol = 2e-2; GEMM + reduce within rtol = atol = 2e-2 (bf16 output) or 1e-3 (fp32 output).
The draws cover what the parametrised tests leave between their grid points: odd world sizes,
row lengths that are not powers of two, sizes on either side of the rules that choose a kernel
variant, ragged GEMM edges, bands that start inside a tile."""
import random

import pytest
import torch

from kraken_amd import comm, fused
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
TOL = dict(rtol=2e-2, atol=2e-2)


def same_bits(a, b):
    return torch.equal(a.cpu().contiguous().view(torch.int16), b.cpu().contiguous().view(torch.int16))


def assert_one_ulp(got, want):
    g, w = got.cpu().float(), want.float()
    d = (g - w).abs()
    assert (d <= w.abs() * 2.0 ** -7 + 1e-30).all(), float(d.max())


@pytest.mark.parametrize("seed", range(24))
def test_reduce_random_shapes(dev, seed):
    rnd = random.Random(1000 + seed)
    W = rnd.choice([1, 2, 3, 4, 5, 6, 7, 8, 8, 8, 16])
    rows = rnd.choice([1, 2, 3, 7, 16, 33, 64, 129, 500])
    D = 8 * rnd.randint(1, 1100)
    stack = orc.make_stack(W, (rows, D), seed0=seed)
    sd = stack.to(dev)
    assert same_bits(comm.one_shot_all_reduce(sd), orc.reduce(stack)), (W, rows, D)
    mode = rnd.choice(["full", "vector"])
    bias = orc.randn_bf16((rows, D) if mode == "full" else (D,), 7 + seed)
    out = torch.empty(rows, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias(sd, None, bias.to(dev), out)
    assert same_bits(out, orc.reduce(stack, bias, bias_first=True)), (W, rows, D, mode)
    # the pointer-table form reads W separate allocations, one of them the caller's own input
    x = orc.randn_bf16((rows, D), 99 + seed)
    rank = rnd.randrange(W)
    bufs = [stack[r].to(dev) for r in range(W)]
    out2 = torch.empty(rows, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias(bufs, x.to(dev), bias.to(dev), out2, rank=rank)
    staged = stack.clone()
    staged[rank] = x
    assert same_bits(out2, orc.reduce(staged, bias, bias_first=True)), (W, rows, D, mode, rank)


@pytest.mark.parametrize("seed", range(32))
def test_reduce_bias_rms_norm_random_shapes(dev, seed):
    rnd = random.Random(2000 + seed)
    W = rnd.choice([1, 2, 3, 4, 5, 7, 8, 8, 8, 16])
    # row lengths on either side of the row kernels' rules: short rows that share a workgroup, one row per
    # workgroup, rows split over several workgroups (long rows, few of them), rows beyond one workgroup's registers
    D = 8 * rnd.choice([1, 5, 40, 125, 512, 640, 767, 768, 769, 1024, 1536, 2048, 3000, 4096, 8192])
    rows = rnd.choice([1, 2, 3, 8, 15, 16, 17, 31, 32, 33, 64, 65, 100])
    if rows * D > 2_000_000:
        rows = max(1, 2_000_000 // D)
    eps = rnd.choice([1e-5, 1e-6, 1e-2])
    stack = orc.make_stack(W, (rows, D), seed0=3 * seed)
    w = orc.randn_bf16((D,), 5 + seed, 0.02, 1.0)
    bias = rnd.choice([None, orc.randn_bf16((rows, D), 7 + seed), orc.randn_bf16((D,), 7 + seed, 0.02)])
    y = torch.empty(rows, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias_rms_norm(stack.to(dev), None, None if bias is None else bias.to(dev), w.to(dev), y,
                                            eps=eps)
    want = orc.reduce_bias_rms_norm(stack, bias, w, eps)
    torch.testing.assert_close(y.cpu(), want, **TOL)
    assert_one_ulp(y, want)
    # a second call on the same stream shares the row-exchange workspace with the first
    y2 = torch.empty_like(y)
    fused.one_shot_all_reduce_bias_rms_norm(stack.to(dev), None, None if bias is None else bias.to(dev), w.to(dev), y2,
                                            eps=eps)
    assert same_bits(y, y2), (W, rows, D)
    x = stack[0] if W == 1 else None
    if x is not None:
        assert_one_ulp(fused.rms_norm(x.to(dev), w.to(dev), eps), orc.rms_norm(x, w, eps))


@pytest.mark.parametrize("seed", range(24))
def test_gemm_reduce_random_shapes(dev, seed):
    rnd = random.Random(3000 + seed)
    M = rnd.choice([8, 40, 128, 200, 256, 264, 512, 520, 777, 1024, 1536])
    N = 8 * rnd.choice([1, 9, 16, 32, 33, 64, 65, 100, 128, 160])
    K = rnd.choice([8, 24, 64, 72, 128, 192, 256, 320, 512, 1000, 2048])
    P = rnd.choice([0, 1, 3, 7])
    b_t = rnd.random() < 0.5
    a = orc.randn_bf16((M, K), 42 + seed)
    b = orc.randn_bf16((N, K), 43 + seed, 0.05).T if b_t else orc.randn_bf16((K, N), 43 + seed, 0.05)
    peers = torch.stack([orc.randn_bf16((M, N), 100 + j + seed) for j in range(P)]) if P else None
    bias = orc.randn_bf16((N,), 5 + seed, 0.02) if rnd.random() < 0.6 else None
    pd = None if peers is None else peers.to(dev)
    bd = None if bias is None else bias.to(dev)
    want = orc.gemm_all_reduce(a, b, peers, bias)
    out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=pd, bias=bd)
    torch.testing.assert_close(out.cpu(), want, rtol=1e-3, atol=1e-3)
    outb = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=pd, bias=bd, out_dtype=BF16)
    torch.testing.assert_close(outb.cpu(), want.to(BF16), **TOL)


@pytest.mark.parametrize("seed", range(16))
def test_gemm_reduce_scatter_random_shapes(dev, seed):
    rnd = random.Random(4000 + seed)
    W = rnd.choice([1, 2, 3, 4, 8])
    M = W * rnd.choice([8, 24, 64, 96, 128, 130, 256])
    N = 8 * rnd.choice([2, 16, 32, 33, 64, 96, 128])
    K = rnd.choice([16, 64, 128, 136, 256, 512, 1024])
    rank = rnd.randrange(W)
    b_t = rnd.random() < 0.5
    a = orc.randn_bf16((M, K), 52 + seed)
    b = orc.randn_bf16((N, K), 53 + seed, 0.05).T if b_t else orc.randn_bf16((K, N), 53 + seed, 0.05)
    peers = torch.stack([orc.randn_bf16((M // W, N), 200 + j + seed) for j in range(W - 1)]) if W > 1 else None
    want, c_want = orc.gemm_reduce_scatter(a, b, peers, rank, W)
    c_scratch = torch.full((M, N), float("nan"), dtype=BF16, device=dev)
    out = fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=None if peers is None else peers.to(dev), rank=rank,
                                    c_scratch=c_scratch, world_size=W)
    assert out.shape == (M // W, N)
    torch.testing.assert_close(out.cpu(), want, **TOL)
    other = torch.ones(M, dtype=torch.bool)
    other[rank * (M // W):(rank + 1) * (M // W)] = False
    torch.testing.assert_close(c_scratch.cpu()[other], c_want[other], **TOL)


@pytest.mark.parametrize("seed", range(12))
def test_all_gather_matmul_random_shapes(dev, seed):
    rnd = random.Random(5000 + seed)
    W = rnd.choice([1, 2, 4, 8])
    m = rnd.choice([8, 32, 64, 128, 256])
    K = rnd.choice([64, 128, 256, 512, 1024])
    N = 8 * rnd.choice([4, 16, 32, 48, 64, 128])
    rank = rnd.randrange(W)
    stack = orc.make_stack(W, (m, K), seed0=60 + seed)
    bT = orc.randn_bf16((N, K), 61 + seed, 0.05)
    a_want, c_want = orc.all_gather_matmul(stack, bT.T)
    a_got, c_got = fused.all_gather_matmul(stack.to(dev), bT.to(dev).T, rank=rank)
    assert same_bits(a_got, a_want)
    torch.testing.assert_close(c_got.cpu(), c_want, **TOL)


@pytest.mark.parametrize("seed", range(24))
def test_large_tile_kernel_random_shapes_and_switches(dev, monkeypatch, seed):
    """The 256 x 256 kernel forced on shapes it would not be chosen for, with a random draw of its
    variants: 16x16x32 or 32x32x16 matrix-core blocks, peers added on the matrix cores or in the
    epilogue, either layout of B, ragged edges, a reduce band that starts and ends inside tiles,
    a forced split of the last tiles' K loops."""
    rnd = random.Random(6000 + seed)
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "256")
    monkeypatch.setenv("KRAKEN_AMD_GEMM_MFMA", rnd.choice(["16", "32"]))
    monkeypatch.setenv("KRAKEN_AMD_GEMM_PEERS", rnd.choice(["mfma", "epilogue"]))
    if rnd.random() < 0.3:
        monkeypatch.setenv("KRAKEN_AMD_GEMM_TAILSPLIT", rnd.choice(["2", "3"]))
    W = rnd.choice([1, 2, 4, 8])
    M = W * rnd.choice([32, 64, 65, 128, 160, 256])
    N = 8 * rnd.choice([32, 33, 64, 65, 96, 128])
    K = 64 * rnd.choice([1, 2, 3, 4, 8, 16])
    rank = rnd.randrange(W)
    b_t = rnd.random() < 0.5
    a = orc.randn_bf16((M, K), 72 + seed)
    b = orc.randn_bf16((N, K), 73 + seed, 0.05).T if b_t else orc.randn_bf16((K, N), 73 + seed, 0.05)
    ad, bd = a.to(dev), b.to(dev)
    if rnd.random() < 0.5:
        peers = torch.stack([orc.randn_bf16((M // W, N), 300 + j + seed) for j in range(W - 1)]) if W > 1 else None
        want, c_want = orc.gemm_reduce_scatter(a, b, peers, rank, W)
        c_scratch = torch.full((M, N), float("nan"), dtype=BF16, device=dev)
        out = fused.gemm_reduce_scatter(ad, bd, peers=None if peers is None else peers.to(dev), rank=rank,
                                        c_scratch=c_scratch, world_size=W)
        torch.testing.assert_close(out.cpu(), want, **TOL)
        other = torch.ones(M, dtype=torch.bool)
        other[rank * (M // W):(rank + 1) * (M // W)] = False
        torch.testing.assert_close(c_scratch.cpu()[other], c_want[other], **TOL)
        assert torch.isnan(c_scratch.cpu()[~other].float()).all()
    else:
        P = rnd.choice([0, 1, 7])
        peers = torch.stack([orc.randn_bf16((M, N), 400 + j + seed) for j in range(P)]) if P else None
        bias = orc.randn_bf16((N,), 9 + seed, 0.02) if rnd.random() < 0.6 else None
        pd = None if peers is None else peers.to(dev)
        bsd = None if bias is None else bias.to(dev)
        want = orc.gemm_all_reduce(a, b, peers, bias)
        torch.testing.assert_close(fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=bsd).cpu(), want,
                                   rtol=1e-3, atol=1e-3)
        torch.testing.assert_close(fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=bsd, out_dtype=BF16).cpu(),
                                   want.to(BF16), **TOL)


@pytest.mark.parametrize("seed", range(10))
def test_fp8_kernel_random_shapes(dev, seed):
    """kr_gemm_fp8 on random whole-tile shapes, row strides and result types: small integers and halves, so every
    fp32 sum is exact and the result must equal the product bit for bit (fp8 results: the saturating conversion
    of the exact product); tile counts on either side of a round of 256 compute units, odd and even k-step counts."""
    from kraken_amd import _lib
    fp8 = torch.float8_e4m3fn
    rnd = random.Random(5000 + seed)
    M, N, K = 256 * rnd.randint(1, 12), 256 * rnd.randint(1, 12), 128 * rnd.randint(1, 9)
    lda, ldb = K + 16 * rnd.randint(0, 3), K + 16 * rnd.randint(0, 3)
    g = torch.Generator().manual_seed(seed)
    a = torch.zeros(M, lda).to(fp8)
    b = torch.zeros(N, ldb).to(fp8)
    a[:, :K] = torch.randint(-2, 3, (M, K), generator=g).float().to(fp8)
    b[:, :K] = (torch.randint(-3, 4, (N, K), generator=g).float() * 0.5).to(fp8)
    a[:, K:], b[:, K:] = 3.0, 3.0                 # what lies between the rows must not be read
    exact = a[:, :K].float() @ b[:, :K].float().T
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    ad, bd = a.to(dev), b.to(dev)
    kind = rnd.choice([0, 1, 2])
    dtype = (BF16, torch.float32, fp8)[kind]
    out = torch.empty(M, N, dtype=dtype, device=dev)
    assert lib.kr_gemm_fp8(ad.data_ptr(), lda, bd.data_ptr(), ldb, M, N, K, out.data_ptr(), kind, stream) == 0, (M, N, K)
    want = exact.clamp(-448.0, 448.0).to(fp8) if kind == 2 else exact.to(dtype)
    assert torch.equal(out.cpu().float(), want.float()), (M, N, K, lda, ldb, kind)
