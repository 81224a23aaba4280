"""GPU parity of the bf16 MFMA GEMM with fused reduce(+bias) epilogue against the CPU oracle.
Gate: rtol = atol = 2e-2 for bf16 outputs vs the fp32-accumulated oracle."""
import os

import pytest
import torch

from kraken_amd import _lib, comm, fused
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
TOL = dict(rtol=2e-2, atol=2e-2)


@pytest.fixture(params=["128", "256", "256-epilogue"])
def tile(request, monkeypatch):
    """Force each GEMM kernel in turn: the register-staged kernel with 128x128 tiles; the
    LDS-DMA kernel with 256x256 tiles (shapes it cannot take fall back to the other), with the
    peers' partial sums of whole-band tiles added on the matrix cores (default) or in the
    epilogue."""
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", request.param[:3])
    monkeypatch.setenv("KRAKEN_AMD_GEMM_PEERS", "epilogue" if request.param.endswith("epilogue") else "mfma")
    return request.param


def mk(M, N, K, P, b_t=False, seed=0):
    a = orc.randn_bf16((M, K), 42 + seed)
    if b_t:
        b = orc.randn_bf16((N, K), 43 + seed, 0.05).T          # b.T contiguous
    else:
        b = orc.randn_bf16((K, N), 43 + seed, 0.05)
    peers = torch.stack([orc.randn_bf16((M, N), 100 + j) for j in range(P)]) if P else None
    return a, b, peers


def test_rank_specific_known_answer(dev, tile):
    # test/test_gemm_allreduce.py:92-117 (M=N=K=32, W=4): every element K*(1+2+3+4), at 1e-5
    M = N = K = 32
    a = torch.ones(M, K, dtype=BF16)
    b = torch.ones(K, N, dtype=BF16)
    peers = torch.stack([torch.full((M, N), float((r + 1) * K), dtype=BF16) for r in range(1, 4)])
    out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=peers.to(dev))
    assert out.dtype == torch.float32 and out.shape == (M, N)
    torch.testing.assert_close(out.cpu(), torch.full((M, N), float(K * 10)), rtol=1e-5, atol=1e-5)
    # same with fp32 operands, as the reference test passes them
    out32 = fused.gemm_one_shot_all_reduce_fused(a.float().to(dev), b.float().to(dev), peers=peers.to(dev))
    torch.testing.assert_close(out32.cpu(), torch.full((M, N), float(K * 10)), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("shape", [(512, 256, 128), (256, 256, 256), (128, 128, 64), (384, 640, 192),
                                   (100, 72, 40), (8, 8, 8), (1000, 264, 520)])
@pytest.mark.parametrize("b_t", [False, True])
def test_gemm_all_reduce_shapes(dev, tile, shape, b_t):
    M, N, K = shape
    a, b, peers = mk(M, N, K, 3, b_t)
    bias = orc.randn_bf16((N,), 42, 0.02)
    want = orc.gemm_all_reduce(a, b, peers, bias)
    out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=peers.to(dev), bias=bias.to(dev))
    torch.testing.assert_close(out.cpu(), want, rtol=1e-3, atol=1e-3)      # fp32 out: tight
    outb = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=peers.to(dev), bias=bias.to(dev),
                                                out_dtype=BF16)
    torch.testing.assert_close(outb.cpu(), want.to(BF16), **TOL)
    plain = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev))
    torch.testing.assert_close(plain.cpu(), orc.gemm_all_reduce(a, b), rtol=1e-3, atol=1e-3)


def test_all_gather_matmul_224_column_tiles(dev, monkeypatch):
    """A plain product with transposed-contiguous B whose 256-column tiles leave a partial round of
    compute units takes 256 x 224 tiles (4096 x 3584: 224 tiles against 256): the whole matrix against
    the oracle, and the same bits as the 256-column form (every element sums the same products in the
    same order)."""
    for name in ("TILE", "MFMA", "N224", "PEERS"):   # the rule under test, whatever the caller's environment forces
        monkeypatch.delenv("KRAKEN_AMD_GEMM_" + name, raising=False)
    W, m, K, N = 8, 512, 320, 3584
    assert _lib.gemm_plan(W * m, N, K, True)["kernel"] == "gemm_dtl16n7_kernel"
    stack = orc.make_stack(W, (m, K), seed0=21)
    bT = orc.randn_bf16((N, K), 22, 0.05)
    a_out, c = fused.all_gather_matmul(stack.to(dev), bT.to(dev).T, rank=5)
    _, want = orc.all_gather_matmul(stack, bT.T)
    torch.testing.assert_close(c.cpu().float(), want.float(), **TOL)
    assert torch.equal(a_out.cpu(), stack.reshape(W * m, K))
    # the overlapped form takes the same tiles (a tile waits for its rows' flags before its first load)
    a_g, c_g = fused.all_gather_matmul(stack.to(dev), bT.to(dev).T, rank=5, gather=True, splits_per_rank=2)
    assert torch.equal(c, c_g) and torch.equal(a_g.cpu(), stack.reshape(W * m, K))
    monkeypatch.setenv("KRAKEN_AMD_GEMM_N224", "0")
    assert _lib.gemm_plan(W * m, N, K, True)["kernel"] == "gemm_dtl16_kernel"
    _, c256 = fused.all_gather_matmul(stack.to(dev), bT.to(dev).T, rank=5)
    assert torch.equal(c, c256)
    # forced on where the rule would not pick it (64 tiles of 224 columns: one partial round either way), odd k-step count
    monkeypatch.setenv("KRAKEN_AMD_GEMM_N224", "1")
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "256")
    W, m, K, N = 4, 256, 192, 896
    stack = orc.make_stack(W, (m, K), seed0=23)
    bT = orc.randn_bf16((N, K), 24, 0.05)
    assert _lib.gemm_plan(W * m, N, K, True)["kernel"] == "gemm_dtl16n7_kernel"
    _, c = fused.all_gather_matmul(stack.to(dev), bT.to(dev).T)
    _, want = orc.all_gather_matmul(stack, bT.T)
    torch.testing.assert_close(c.cpu().float(), want.float(), **TOL)


def test_fp8_conversions(dev):
    """kr_cast_fp8_to_bf16 on all 256 codes and kr_cast_f32_to_fp8 on random and boundary values,
    against torch's CPU conversions (nearest even); from magnitude 448 on the result saturates to
    448 where torch gives NaN (from 464 on)."""
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    fp8 = torch.float8_e4m3fn
    codes = torch.arange(256, dtype=torch.uint8).repeat(4)
    out = torch.empty(codes.numel(), dtype=BF16, device=dev)
    assert lib.kr_cast_fp8_to_bf16(codes.to(dev).data_ptr(), codes.numel(), out.data_ptr(), stream) == 0
    want = codes.view(fp8).to(BF16)
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(out.cpu()), nan) and torch.equal(out.cpu()[~nan].view(torch.int16), want[~nan].view(torch.int16))
    g = torch.Generator().manual_seed(3)
    x = torch.cat([torch.randn(1 << 16, generator=g) * s_ for s_ in (1e-3, 0.02, 1.0, 30.0, 300.0)])
    edge = torch.tensor([0.0, -0.0, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -9, 2.5 * 2.0 ** -9, 2.0 ** -6, 0.9375 * 2.0 ** -6,
                         447.9, 448.0, 463.9, 464.0, 1e9, -1e9, float("inf"), -float("inf")])
    x = torch.cat([x, edge, torch.zeros(-(x.numel() + edge.numel()) % 16)])
    y = torch.empty(x.numel(), dtype=torch.uint8, device=dev)
    assert lib.kr_cast_f32_to_fp8(x.to(dev).data_ptr(), x.numel(), y.data_ptr(), stream) == 0
    got = y.cpu()
    small = x.abs() < 448
    assert torch.equal(got[small], x[small].to(fp8).view(torch.uint8))
    assert torch.equal(got[~small] & 0x7f, torch.full_like(got[~small], 0x7e))           # saturated, sign kept
    assert torch.equal(got[~small] >> 7, (x[~small] < 0).to(torch.uint8))
    z = torch.full((16,), float("nan"))
    assert lib.kr_cast_f32_to_fp8(z.to(dev).data_ptr(), 16, y.data_ptr(), stream) == 0
    assert torch.isnan(y.cpu()[:16].view(fp8).float()).all()


def test_all_gather_matmul_fp8(dev):
    """The fp8 branch (kraken/fused/all_gather_matmul.py:53,121,213): fp8 shards and b, fp8 result.
    With small integers and halves every fp32 sum is exact whatever its order, so the result equals
    the oracle bit for bit, saturated elements included; with random operands it is within one fp8
    step of the oracle (the orders of the fp32 sums differ) and mostly equal."""
    fp8 = torch.float8_e4m3fn
    W, m, K, N = 8, 64, 512, 384
    g = torch.Generator().manual_seed(11)
    a = torch.randint(-2, 3, (W, m, K), generator=g).float().to(fp8)
    bT = (torch.randint(-3, 4, (N, K), generator=g).float() * 0.5).to(fp8)
    a_out, c = fused.all_gather_matmul(a.to(dev), bT.to(dev).T, rank=3)
    a_full, want = orc.all_gather_matmul_fp8(a, bT.T)
    assert c.dtype == fp8 and a_out.dtype == fp8
    assert torch.equal(a_out.cpu().view(torch.uint8), a_full.view(torch.uint8))
    assert torch.equal(c.cpu().view(torch.uint8), want.view(torch.uint8))
    # a shape the 256x256 kernel takes, random operands, one fp8 step of slack
    W, m, K, N = 8, 512, 1024, 4096
    a = (torch.randn(W, m, K, generator=g)).to(fp8)
    bT = (torch.randn(N, K, generator=g) * 0.05).to(fp8)
    _, c = fused.all_gather_matmul(a.to(dev), bT.to(dev).T)
    _, want = orc.all_gather_matmul_fp8(a, bT.T)
    got, ref = c.cpu().float(), want.float()
    assert (got == ref).float().mean() > 0.99
    step = torch.maximum(ref.abs(), torch.tensor(2.0 ** -6)) * 2.0 ** -3          # spacing of e4m3 at that magnitude
    assert ((got - ref).abs() <= step).all()


@pytest.mark.parametrize("K", [128, 256, 384, 1024])
def test_fp8_kernel_exact_sums(dev, K):
    """kr_gemm_fp8 (fp8 operands on the fp8 matrix-core instruction): with small integers and halves every
    fp32 sum is exact whatever its order, so all three result types equal the oracle bit for bit -- the fp8
    result with its saturated elements, through the wrapper and straight through the C ABI; one, two, an odd
    number and many k-steps."""
    fp8 = torch.float8_e4m3fn
    W, m, N = 8, 64, 768
    g = torch.Generator().manual_seed(31 + K)
    a = torch.randint(-2, 3, (W, m, K), generator=g).float().to(fp8)
    bT = (torch.randint(-3, 4, (N, K), generator=g).float() * 0.5).to(fp8)
    a[0], a[1], bT[:64] = 4.0, -4.0, 1.5            # sums of +-6K: beyond the largest fp8 value on both sides
    a_full, want = orc.all_gather_matmul_fp8(a, bT.T)
    exact = a.reshape(W * m, K).float() @ bT.float().T
    assert (exact > 448).any() and (exact < -448).any() and (exact.abs() < 448).any()      # the case has saturating and ordinary sums
    a_out, c = fused.all_gather_matmul(a.to(dev), bT.to(dev).T, rank=2)
    assert c.dtype == fp8 and torch.equal(a_out.cpu().view(torch.uint8), a_full.view(torch.uint8))
    assert torch.equal(c.cpu().view(torch.uint8), want.view(torch.uint8))
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    ad, bd = a.reshape(W * m, K).to(dev), bT.to(dev)
    for kind, dtype in ((1, torch.float32), (0, BF16)):
        out = torch.full((W * m, N), 7, dtype=dtype, device=dev)
        assert lib.kr_gemm_fp8(ad.data_ptr(), K, bd.data_ptr(), K, W * m, N, K, out.data_ptr(), kind, stream) == 0
        assert torch.equal(out.cpu(), exact.to(dtype))


def test_fp8_kernel_random_operands_and_nan(dev):
    """Random operands: within one fp8 step of the oracle and of the widening path (the orders of the fp32
    sums differ), mostly equal; the fp32 result against a double-precision product; row strides larger than
    K; a NaN operand element makes its row of the result NaN and nothing else."""
    fp8 = torch.float8_e4m3fn
    W, m, K, N = 8, 128, 2048, 1280
    g = torch.Generator().manual_seed(41)
    a = torch.randn(W, m, K, generator=g).to(fp8)
    bT = (torch.randn(N, K, generator=g) * 0.05).to(fp8)
    _, c = fused.all_gather_matmul(a.to(dev), bT.to(dev).T)
    _, c_wide = fused.all_gather_matmul(a.to(dev), bT.to(dev).T, fp8_kernel=False)
    _, want = orc.all_gather_matmul_fp8(a, bT.T)
    ref = want.float()
    step = torch.maximum(ref.abs(), torch.tensor(2.0 ** -6)) * 2.0 ** -3          # spacing of e4m3 at that magnitude
    for got in (c.cpu().float(), c_wide.cpu().float()):
        assert (got == ref).float().mean() > 0.99
        assert ((got - ref).abs() <= step).all()
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    M = W * m
    a_pad = torch.zeros(M, K + 64, dtype=torch.uint8).view(fp8)
    a_pad[:, :K] = a.reshape(M, K)
    b_pad = torch.zeros(N, K + 16, dtype=torch.uint8).view(fp8)
    b_pad[:, :K] = bT
    ad, bd = a_pad.to(dev), b_pad.to(dev)
    out = torch.empty(M, N, dtype=torch.float32, device=dev)
    assert lib.kr_gemm_fp8(ad.data_ptr(), K + 64, bd.data_ptr(), K + 16, M, N, K, out.data_ptr(), 1, stream) == 0
    exact = (a.reshape(M, K).double() @ bT.double().T)
    torch.testing.assert_close(out.cpu().double(), exact, rtol=1e-5, atol=1e-3)      # fp32 sums of 2048 products of size 0.05
    a_nan = a.reshape(M, K).clone()
    a_nan.view(torch.uint8)[300, 77] = 0x7f
    c = torch.empty(M, N, dtype=fp8, device=dev)
    assert lib.kr_gemm_fp8(a_nan.to(dev).data_ptr(), K, bT.to(dev).data_ptr(), K, M, N, K, c.data_ptr(), 2, stream) == 0
    nan = torch.isnan(c.cpu().float())
    assert nan[300].all() and not nan[:300].any() and not nan[301:].any()


@pytest.mark.parametrize("splits", [1, 2])
@pytest.mark.parametrize("as_list", [False, True])
def test_all_gather_matmul_fp8_overlapped(dev, splits, as_list):
    """gather=True with fp8 shards (the reference's overlap, all_gather_matmul.py:308-323, on its fp8 branch):
    the chunks are copied on the side stream and flagged while the fp8 kernel's tiles wait for them; the
    gathered matrix is the shards bit for bit, every flag ends at 1, and the product has the bits of the
    gather=False call (same kernel, same sums).  Also a shape the fp8 kernel does not take (the widening
    path behind the finished gather)."""
    from kraken_amd import _waits
    fp8 = torch.float8_e4m3fn
    W, m, K, N = 8, 256, 1024, 768
    g = torch.Generator().manual_seed(51)
    a = torch.randn(W, m, K, generator=g).to(fp8)
    bT = (torch.randn(N, K, generator=g) * 0.05).to(fp8)
    ad, bd = a.to(dev), bT.to(dev)
    _, want = fused.all_gather_matmul(ad, bd.T, rank=5)
    shards = [ad[r].clone() for r in range(W)] if as_list else ad
    progress = torch.zeros(W * splits, dtype=torch.int32, device=dev)
    a_out, c = fused.all_gather_matmul(shards, bd.T, None, progress, rank=5, splits_per_rank=splits, gather=True)
    torch.cuda.synchronize()
    _waits.check(block=True)
    assert a_out.dtype == fp8 and torch.equal(a_out.cpu().view(torch.uint8), a.reshape(W * m, K).view(torch.uint8))
    assert (progress.cpu() == 1).all()
    assert torch.equal(c.cpu().view(torch.uint8), want.cpu().view(torch.uint8))
    _, ref = orc.all_gather_matmul_fp8(a, bT.T)
    assert (c.cpu().float() == ref.float()).float().mean() > 0.99
    # 8 x 48 rows: not a multiple of 256
    a2, b2 = a[:, :48].contiguous(), bT[:400]
    a_out, c = fused.all_gather_matmul(a2.to(dev), b2.to(dev).T, rank=1, gather=True)
    _, ref = orc.all_gather_matmul_fp8(a2, b2.T)
    assert torch.equal(a_out.cpu().view(torch.uint8), a2.reshape(-1, K).view(torch.uint8))
    assert (c.cpu().float() == ref.float()).float().mean() > 0.99


def test_split_fp32_is_one_pass_and_bit_exact(dev):
    """kr_split_fp32 writes the hi / lo blocks of an fp32 operand in the three layouts the GEMM
    wrappers use, bit for bit what elementwise torch ops give (hi = bf16(x), lo = bf16(x - hi)),
    also for a row stride larger than the row."""
    from kraken_amd.fused import _gemm
    g = torch.Generator().manual_seed(7)
    for (M, K, N) in [(64, 128, 72), (300, 264, 136), (8, 8, 8)]:
        a = torch.randn(M, K + 8, generator=g).to(dev)[:, :K]            # row stride K + 8
        b = torch.randn(K, N, generator=g).to(dev)
        bt = torch.randn(N, K, generator=g).to(dev).T                     # transposed-contiguous [K, N]
        for (x, y) in ((a, b), (a, bt)):
            a3, b3 = _gemm.split_fp32(x, y)
            x_hi = x.to(BF16); x_lo = (x - x_hi.float()).to(BF16)
            y_hi = y.to(BF16); y_lo = (y - y_hi.float()).to(BF16)
            assert torch.equal(a3, torch.cat([x_hi, x_hi, x_lo], dim=1))
            assert torch.equal(b3, torch.cat([y_hi, y_lo, y_hi], dim=0))
            assert b3.T.is_contiguous() == (y is bt)                      # the operand's layout is kept
            # the 3K-long bf16 product is a @ b to ~16 mantissa bits
            ref = x.double() @ y.double()
            got = (a3.double() @ b3.double())
            assert (got - ref).abs().max() <= 2e-4 * ref.abs().max() + 1e-6
    # sizes the kernel does not take fall back to elementwise ops with the same result
    a = torch.randn(16, 12, generator=g).to(dev); b = torch.randn(12, 20, generator=g).to(dev)
    a3, b3 = _gemm.split_fp32(a, b)
    assert a3.shape == (16, 36) and b3.shape == (36, 20)
    assert torch.equal(a3[:, :12], a.to(BF16)) and torch.equal(b3[12:24], (b - b.to(BF16).float()).to(BF16))


def test_fp32_operands_reference_shapes(dev, tile):
    # test/test_gemm_allreduce.py:51-89: fp32 N(0,1) operands, (512,256,128) and (256,256,256), tol 1e-1
    for (M, N, K) in [(512, 256, 128), (256, 256, 256)]:
        g = torch.Generator().manual_seed(42)
        a = torch.randn(M, K, generator=g)
        b = torch.randn(K, N, generator=g)
        out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev))
        torch.testing.assert_close(out.cpu(), a @ b, rtol=1e-1, atol=1e-1)
        torch.testing.assert_close(out.cpu(), a @ b, rtol=2e-3, atol=2e-3)   # the split keeps ~16 bits


@pytest.mark.parametrize("rank", [0, 2, 3])
@pytest.mark.parametrize("b_t", [False, True])
def test_gemm_reduce_scatter(dev, tile, rank, b_t):
    M, N, K, W = 512, 256, 128, 4        # test/test_gemm_reduce_scatter.py:61-74
    a, b, _ = mk(M, N, K, 0, b_t)
    peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(W - 1)])
    want, c_want = orc.gemm_reduce_scatter(a, b, peers, rank, W)
    c_scratch = torch.full((M, N), float("nan"), dtype=BF16, device=dev)
    out = fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=peers.to(dev), rank=rank, c_scratch=c_scratch)
    assert out.shape == (M // W, N) and out.dtype == BF16
    torch.testing.assert_close(out.cpu(), want, **TOL)
    rows = torch.ones(M, dtype=torch.bool)
    rows[rank * M // W:(rank + 1) * M // W] = False
    torch.testing.assert_close(c_scratch.cpu()[rows], c_want[rows], **TOL)
    assert torch.isnan(c_scratch.cpu()[~rows].float()).all()    # own band never makes the round trip


def test_gemm_reduce_scatter_rank_specific(dev, tile):
    # test/test_gemm_reduce_scatter.py:76-91
    M, N, K, W = 512, 256, 128, 4
    for rank in range(W):
        a = torch.full((M, K), float(rank + 1), dtype=BF16)
        b = torch.ones(K, N, dtype=BF16)
        others = [r for r in range(W) if r != rank]
        peers = torch.stack([torch.full((M // W, N), float((r + 1) * K), dtype=BF16) for r in others])
        out = fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=peers.to(dev), rank=rank)
        assert torch.equal(out.cpu().float(), torch.full((M // W, N), float(K * 10)))


@pytest.mark.parametrize("rank", [0, 3])
def test_all_gather_matmul(dev, tile, rank):
    W, m, K, N = 4, 128, 256, 384
    stack = orc.make_stack(W, (m, K))
    bT = orc.randn_bf16((N, K), 43, 0.05)
    sd = stack.to(dev)
    progress = torch.zeros(W, dtype=torch.int32, device=dev)
    ag, c = fused.all_gather_matmul(sd, bT.to(dev).T, progress=progress, rank=rank)
    a_want, c_want = orc.all_gather_matmul(stack, bT.T)
    assert torch.equal(ag.cpu(), a_want)                      # test/test_allgather_matmul.py:75: exact
    assert ag.data_ptr() == sd.data_ptr()                     # zero-copy view
    assert (progress != 0).all()                              # test/test_allgather.py:73
    torch.testing.assert_close(c.cpu(), c_want, **TOL)
    a_out = torch.empty(W * m, K, dtype=BF16, device=dev)
    ag2, c2 = fused.all_gather_matmul(sd, bT.to(dev).T, a_out=a_out, rank=rank)
    assert ag2 is a_out and torch.equal(a_out.cpu(), a_want) and torch.equal(c2, c)


@pytest.mark.parametrize("rank,splits", [(0, 1), (2, 2), (3, 4)])
@pytest.mark.parametrize("as_list", [False, True])
def test_all_gather_matmul_overlapped_with_the_copies(dev, tile, rank, splits, as_list):
    """The reference's overlap: chunk copies with arrival flags on a side stream, tiles that
    wait for their chunk (kraken/fused/all_gather_matmul.py:95-110); local shard read in place."""
    W, m, K, N = 4, 256, 320, 384
    stack = orc.make_stack(W, (m, K), seed0=7)
    bT = orc.randn_bf16((N, K), 43, 0.05)
    a_want, c_want = orc.all_gather_matmul(stack, bT.T)
    shards = [stack[r].to(dev) for r in range(W)] if as_list else stack.to(dev)
    progress = torch.full((W * splits,), 7, dtype=torch.int32, device=dev)       # stale values: must be reset
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    a_out = torch.full((W * m, K), float("nan"), dtype=BF16, device=dev)
    ag, c = fused.all_gather_matmul(shards, bT.to(dev).T, a_out=a_out, progress=progress, rank=rank,
                                    splits_per_rank=splits, gather=True, status=status)
    torch.cuda.synchronize()
    assert ag is a_out and torch.equal(ag.cpu(), a_want)          # test/test_allgather_matmul.py:75: exact
    assert (progress == 1).all()                                  # test/test_allgather.py:73
    assert status.item() == 0
    torch.testing.assert_close(c.cpu(), c_want, **TOL)
    # same bits as the GEMM on the already gathered matrix
    _, c_plain = fused.all_gather_matmul(stack.to(dev), bT.to(dev).T, rank=rank)
    assert torch.equal(c, c_plain)


def test_all_gather_w_progress(dev):
    # test/test_allgather.py:50-75: gathered tensor exact, every flag set
    W, m, K = 8, 64, 128
    stack = orc.make_stack(W, (m, K), seed0=3)
    for splits, rank in ((1, 0), (4, 5)):
        progress = torch.zeros(W * splits, dtype=torch.int32, device=dev)
        out = comm.all_gather_w_progress([stack[r].to(dev) for r in range(W)], progress=progress,
                                         splits_per_rank=splits, rank=rank)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), stack.reshape(W * m, K))
        assert (progress == 1).all()


def test_all_gather_matmul_wait_is_bounded(dev, tile):
    """A flag that never comes: every tile's wait ends at the limit, the kernel exits and the
    status names a chunk (no copy is enqueued here; the limit is 2 ms)."""
    from kraken_amd.fused.all_gather_matmul import _matmul_w_progress
    W, m, K, N = 4, 256, 128, 256
    a = orc.randn_bf16((W * m, K), 1).to(dev)
    bT = orc.randn_bf16((N, K), 2, 0.05).to(dev)
    progress = torch.zeros(W, dtype=torch.int32, device=dev)
    progress[1] = 1                                               # one chunk present, two missing
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    cfg = {"RANK": 0, "WORLD_SIZE": W, "SPLITS_PER_RANK": 1, "wait_limit_us": 2000}
    c = _matmul_w_progress(a, a[:m], bT.T, progress, cfg, status)
    torch.cuda.synchronize()
    assert status.item() in (3, 4)                                # 1 + index of a missing chunk
    want = (a.float().cpu() @ bT.float().cpu().T).to(BF16)
    torch.testing.assert_close(c[:2 * m].cpu(), want[:2 * m], **TOL)   # local shard and the present chunk
    # with every flag set the same call is complete and the status stays clear
    progress.fill_(1)
    status.zero_()
    c = _matmul_w_progress(a, a[:m], bT.T, progress, cfg, status)
    torch.cuda.synchronize()
    assert status.item() == 0
    torch.testing.assert_close(c.cpu(), want, **TOL)


def test_ce_persistent_variant(dev, tile):
    M, N, K, W = 512, 256, 128, 4
    a, b, _ = mk(M, N, K, 0, True)
    for rank in (0, 2):
        peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(W - 1)])
        out = fused.gemm_reduce_scatter_ce_persistent(a.to(dev), b.to(dev), peers=peers.to(dev), rank=rank)
        c = (a.float() @ b.float()).to(BF16)
        bands = list(peers)
        bands.insert(rank, c[rank * M // W:(rank + 1) * M // W])
        want = orc.reduce_rotated(torch.cat(bands, 0), W, rank, acc_bf16=True)
        torch.testing.assert_close(out.cpu(), want, **TOL)


def test_split_k_loop_replays_from_a_graph(dev):
    """The GEMM entry points enqueue kernels only (the split K loop included: partial products,
    then the finishing pass): captured once, every replay reproduces the eager result bit for
    bit, with eager work between the replays."""
    M, N, K, W = 512, 256, 128, 4
    a, b, peers = mk(M, N, K, 3, True)
    bias = orc.randn_bf16((N,), 42, 0.02)
    ad, bd, pd, biasd = a.to(dev), b.to(dev), peers.to(dev), bias.to(dev)
    band_peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(W - 1)]).to(dev)
    c_scratch = torch.zeros(M, N, dtype=BF16, device=dev)       # (the own band's rows are never written)
    stack = orc.make_stack(W, (M // W, K)).to(dev)
    a_few, b_few, _ = mk(128, 384, 1024, 0, False, seed=9)       # 3 tiles: its K loop is split
    a_few, b_few = a_few.to(dev), b_few.to(dev)
    assert _lib.load().kr_gemm_workspace_bytes(128, 384, 1024) > 0

    def run():
        o1 = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=biasd)
        o2 = fused.gemm_reduce_scatter(ad, bd, peers=band_peers, rank=1, c_scratch=c_scratch)
        _, o3 = fused.all_gather_matmul(stack, bd, rank=2)
        o4 = fused.gemm_one_shot_all_reduce_fused(a_few, b_few)
        return o1, o2, c_scratch, o3, o4

    eager = [t.clone() for t in run()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        run()                                   # the stream's workspace exists before the capture
        side.synchronize()
        with torch.cuda.graph(g, stream=side):
            got = run()
    for rep in range(3):
        for t in got:
            t.zero_()
        _ = fused.gemm_one_shot_all_reduce_fused(a_few, b_few)   # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for e, r in zip(eager, got):
            assert torch.equal(e, r)


@pytest.mark.parametrize("b_t", [False, True])
def test_both_mfma_block_shapes_agree(dev, monkeypatch, b_t):
    """The 256 x 256 kernel's k loop on 16x16x32 blocks (default) and on 32x32x16 blocks: the same
    products, summed 32 or 16 at a time inside the matrix cores, so the fp32 results agree to
    rounding and the bf16 ones to an ulp -- for full and ragged shapes, the reduce-scatter form
    and the split launches."""
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "256")
    outs = {}
    for mfma in ("16", "32"):
        monkeypatch.setenv("KRAKEN_AMD_GEMM_MFMA", mfma)
        res = []
        for (M, N, K) in [(512, 768, 448), (520, 264, 192), (256, 256, 64)]:
            a, b, _ = mk(M, N, K, 0, b_t, seed=K)
            ad, bd = a.to(dev), b.to(dev)
            res.append(fused.gemm_one_shot_all_reduce_fused(ad, bd))
            res.append(fused.gemm_one_shot_all_reduce_fused(ad, bd, out_dtype=BF16))
        M, N, K, W = 1024, 512, 256, 4
        a, b, _ = mk(M, N, K, 0, b_t, seed=1)
        peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(W - 1)]).to(dev)
        c_scratch = torch.zeros(M, N, dtype=BF16, device=dev)
        res.append(fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=peers, rank=2, c_scratch=c_scratch))
        res.append(c_scratch)
        monkeypatch.setenv("KRAKEN_AMD_GEMM_TAILSPLIT", "4")      # 6 tiles, every one split four ways
        a, b, _ = mk(512, 768, 1024, 0, b_t, seed=2)
        res.append(fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev)))
        monkeypatch.delenv("KRAKEN_AMD_GEMM_TAILSPLIT")
        outs[mfma] = res
    for x, y in zip(outs["16"], outs["32"]):
        if x.dtype == torch.float32:
            torch.testing.assert_close(x, y, rtol=1e-5, atol=1e-4)
        else:
            # two bf16 ulps: in the reduce-scatter form the 32x32x16 kernel adds the band's peers on
            # the matrix cores (one rounding), the 16x16x32 kernel in the epilogue (product rounded first)
            torch.testing.assert_close(x, y, rtol=1.6e-2, atol=1e-2)
    a, b, _ = mk(512, 768, 448, 0, b_t, seed=448)
    torch.testing.assert_close(outs["16"][0].cpu(), a.float() @ b.float(), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("b_t", [False, True])
@pytest.mark.parametrize("mfma", ["16", "32"])
def test_split_parts_of_very_few_k_steps(dev, monkeypatch, b_t, mfma):
    """Forced splits that leave a workgroup one or two k-steps (and uneven shares): the prologue,
    the loads past the end and the waits of the k loop must still line up."""
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "256")
    monkeypatch.setenv("KRAKEN_AMD_GEMM_MFMA", mfma)
    for (M, N, K, S) in [(512, 768, 256, 4), (512, 768, 192, 3), (256, 256, 64, 1), (512, 512, 128, 2), (768, 512, 320, 5),
                         (512, 768, 448, 2)]:
        monkeypatch.setenv("KRAKEN_AMD_GEMM_TAILSPLIT", str(S))
        a, b, _ = mk(M, N, K, 0, b_t, seed=S)
        out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev))
        torch.testing.assert_close(out.cpu(), a.float() @ b.float(), rtol=1e-3, atol=1e-3)


def _band_tile_counts(M, N, W, bm):
    rows = M // W
    return [(((r + 1) * rows - 1) // bm - (r * rows) // bm + 1) * -(-N // bm) for r in range(W)]


@pytest.mark.parametrize("shape,W,rank", [((512, 256, 128), 4, 1), ((768, 384, 192), 3, 2), ((1024, 512, 256), 8, 7),
                                          ((1000, 264, 512), 4, 0), ((1000, 264, 520), 4, 3)])
def test_producer_gemm_flags_every_band(dev, tile, shape, W, rank):
    """Producer GEMM of the copy-engine reduce-scatter: all of C, one counter and one flag per
    destination rank's band (bands that start inside a tile included)."""
    from kraken_amd.fused.gemm_reduce_scatter_ce_persistent import gemm_producer_w_progress
    M, N, K = shape
    a, b, _ = mk(M, N, K, 0, True, seed=W)
    gemm_out = torch.full((M, N), float("nan"), dtype=BF16, device=dev)
    progress = torch.zeros(W, dtype=torch.int32, device=dev)
    signal_pad = torch.zeros(W, dtype=torch.int32, device=dev)
    gemm_producer_w_progress(a.to(dev), b.to(dev), gemm_out, progress, signal_pad, {"RANK": rank, "WORLD_SIZE": W})
    torch.cuda.synchronize()
    assert signal_pad.tolist() == [1] * W
    assert progress.tolist() in (_band_tile_counts(M, N, W, 128), _band_tile_counts(M, N, W, 256))
    torch.testing.assert_close(gemm_out.cpu(), (a.float() @ b.float()).to(BF16), **TOL)


def test_producer_gemm_counts_bands_of_a_shape_with_a_partial_last_round(dev):
    """272 tiles of 256 x 256 = one round of the compute units and a partial second one: the plain GEMM
    would split that tail over idle compute units (a workspace is asked for), the producer keeps the
    one-pass kernel so that every band is counted and flagged when it is finished."""
    from kraken_amd import _lib
    from kraken_amd.fused.gemm_reduce_scatter_ce_persistent import gemm_producer_w_progress
    M, N, K, W, rank = 4352, 4096, 4096, 8, 3
    assert _lib.load().kr_gemm_workspace_bytes(M, N, K) > 0
    g = torch.Generator().manual_seed(11)
    a = (torch.randn(M, K, generator=g) * 0.25).to(BF16)
    b = (torch.randn(K, N, generator=g) * 0.25).to(BF16)
    gemm_out = torch.full((M, N), float("nan"), dtype=BF16, device=dev)
    progress = torch.zeros(W, dtype=torch.int32, device=dev)
    signal_pad = torch.zeros(W, dtype=torch.int32, device=dev)
    gemm_producer_w_progress(a.to(dev), b.to(dev), gemm_out, progress, signal_pad, {"RANK": rank, "WORLD_SIZE": W})
    torch.cuda.synchronize()
    assert signal_pad.tolist() == [1] * W
    assert progress.tolist() == _band_tile_counts(M, N, W, 256)
    torch.testing.assert_close(gemm_out.cpu(), (a.float() @ b.float()).to(BF16), **TOL)


@pytest.mark.parametrize("rank", [0, 2])
def test_copy_engine_scatter_overlaps_the_producer(dev, tile, rank):
    """The reference's overlap: the band copies sit on a side stream behind stream-ordered waits
    for the producer's flags (kraken/fused/gemm_reduce_scatter_ce_persistent.py:137-175,343-370)."""
    from kraken_amd.fused.gemm_reduce_scatter_ce_persistent import gemm_producer_w_progress
    M, N, K, W = 2048, 1024, 256, 4
    a, b, _ = mk(M, N, K, 0, True, seed=3)
    peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(W - 1)])
    sent = torch.full((W, M // W, N), float("nan"), dtype=BF16, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    out = fused.gemm_reduce_scatter_ce_persistent(a.to(dev), b.to(dev), peers=peers.to(dev), rank=rank, sent=sent,
                                                  status=status)
    torch.cuda.synchronize()
    assert status.item() == 0
    c = (a.float() @ b.float()).to(BF16)
    bands = list(peers)
    bands.insert(rank, c[rank * M // W:(rank + 1) * M // W])
    want = orc.reduce_rotated(torch.cat(bands, 0), W, rank, acc_bf16=True)
    torch.testing.assert_close(out.cpu(), want, **TOL)
    # every other rank's band went out as the GEMM wrote it; the own band went to the scatter buffer
    gemm_out = torch.empty(M, N, dtype=BF16, device=dev)
    progress = torch.zeros(W, dtype=torch.int32, device=dev)
    signal_pad = torch.zeros(W, dtype=torch.int32, device=dev)
    gemm_producer_w_progress(a.to(dev), b.to(dev), gemm_out, progress, signal_pad, {"RANK": rank, "WORLD_SIZE": W})
    for r in range(W):
        if r != rank:
            assert torch.equal(sent[r], gemm_out[r * M // W:(r + 1) * M // W])
        else:
            assert torch.isnan(sent[r].float()).all()
    assert torch.equal(out, fused.gemm_reduce_scatter_ce_persistent(a.to(dev), b.to(dev), peers=peers.to(dev), rank=rank))


def test_copies_on_the_copy_engines(dev):
    """copy_engine=True: the chunk copies of the all-gather and the band copies of the scatter go
    through kr_copy_engine_memcpy (SDMA) instead of copy kernels; same bits either way."""
    from kraken_amd.fused.gemm_reduce_scatter_ce_persistent import copy_engine_scatter, gemm_producer_w_progress
    W, m, K, N = 4, 256, 512, 384
    stack = orc.make_stack(W, (m, K), seed0=11)
    bT = orc.randn_bf16((N, K), 43, 0.05)
    shards = [stack[r].to(dev) for r in range(W)]
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    a_out = torch.full((W * m, K), float("nan"), dtype=BF16, device=dev)
    ag, c = fused.all_gather_matmul(shards, bT.to(dev).T, a_out=a_out, rank=1, splits_per_rank=2, copy_engine=True,
                                    status=status)
    torch.cuda.synchronize()
    assert status.item() == 0 and torch.equal(ag.cpu(), stack.reshape(W * m, K))
    assert torch.equal(c, fused.all_gather_matmul(stack.to(dev), bT.to(dev).T)[1])
    gemm_out = torch.empty(W * m, N, dtype=BF16, device=dev)
    progress = torch.zeros(W, dtype=torch.int32, device=dev)
    signal_pad = torch.zeros(W, dtype=torch.int32, device=dev)
    gemm_producer_w_progress(ag, bT.to(dev).T, gemm_out, progress, signal_pad, {"RANK": 2, "WORLD_SIZE": W})
    sent = torch.zeros(W, m, N, dtype=BF16, device=dev)
    copy_engine_scatter(gemm_out, sent, signal_pad, rank=2, status=status, copy_engine=True)
    torch.cuda.synchronize()
    assert status.item() == 0 and torch.equal(sent.view(W * m, N), gemm_out)


def test_flag_arrive_wait(dev):
    """test/test_ptx_utils.py:80-116: 8 producer workgroups set their flags, 32 consumers wait for
    them in the same launch; the flags end as 1 and no consumer runs into the limit."""
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    flags = torch.zeros(64, dtype=torch.int32, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    _lib.check(lib.kr_flag_arrive_wait(flags.data_ptr(), 8, 32, 0, status.data_ptr(), stream), "flag_arrive_wait")
    torch.cuda.synchronize()
    expect = torch.zeros_like(flags)
    expect[:8] = 1
    assert torch.equal(flags, expect) and status.item() == 0
    # one producer, four consumers, on a flag further into the array
    flags.zero_()
    _lib.check(lib.kr_flag_arrive_wait(flags.data_ptr() + 4, 1, 4, 2000, status.data_ptr(), stream), "flag_arrive_wait")
    torch.cuda.synchronize()
    assert flags.tolist() == [0, 1] + [0] * 62 and status.item() == 0


def test_copy_engine_scatter_wait_is_bounded(dev):
    """A flag that never comes: the stream-ordered wait gives up after its limit, records it in
    `status`, and the stream drains."""
    from kraken_amd.fused.gemm_reduce_scatter_ce_persistent import copy_engine_scatter
    W, rows, N = 2, 64, 128
    inp = torch.ones(W * rows, N, dtype=BF16, device=dev)
    signal_pad = torch.tensor([1, 0], dtype=torch.int32, device=dev)      # band 1 is never flagged
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    outs = [torch.zeros(rows, N, dtype=BF16, device=dev) for _ in range(W)]
    copy_engine_scatter(inp, outs, signal_pad, rank=0, wait_limit_us=2000, status=status)
    torch.cuda.synchronize()
    assert status.item() == 1
    ok = torch.zeros(1, dtype=torch.int32, device=dev)
    copy_engine_scatter(inp, [outs[0], None], torch.ones(W, dtype=torch.int32, device=dev), rank=1,
                        wait_limit_us=2000, status=ok)
    torch.cuda.synchronize()
    assert ok.item() == 0 and torch.equal(outs[0], inp[:rows])


def test_bounded_waits_without_a_status_do_not_fail_silently(dev):
    """No `status` passed: the wrappers keep a word of their own, every wait of the call shares it
    (after the first one runs out the others give up at once), and the failure is raised on the
    next look -- here by an explicit check, in use by the next call of an overlap function."""
    import time
    from kraken_amd import _waits
    from kraken_amd._lib import KrakenAmdError
    from kraken_amd.fused.gemm_reduce_scatter_ce_persistent import copy_engine_scatter
    W, rows, N = 8, 64, 128
    inp = torch.ones(W * rows, N, dtype=BF16, device=dev)
    outs = [torch.zeros(rows, N, dtype=BF16, device=dev) for _ in range(W)]
    _waits.check(block=True)                                              # nothing pending from earlier tests
    copy_engine_scatter(inp, outs, torch.ones(W, dtype=torch.int32, device=dev), rank=0)      # every flag is set
    _waits.check(block=True)
    never = torch.zeros(W, dtype=torch.int32, device=dev)                 # no flag ever comes: 8 waits of 20 ms
    t0 = time.perf_counter()
    copy_engine_scatter(inp, outs, never, rank=0, wait_limit_us=20000)
    with pytest.raises(KrakenAmdError, match="ran out in.*copy_engine_scatter"):
        _waits.check(block=True)
    assert time.perf_counter() - t0 < 0.1                                 # one limit, not eight
    _waits.check(block=True)                                              # reported once
    # two failing calls before anybody looks: both are named (the second gives up at once: the
    # stream's word is still set when its waits start)
    t0 = time.perf_counter()
    copy_engine_scatter(inp, outs, never, rank=0, wait_limit_us=20000)
    copy_engine_scatter(inp, outs, never, rank=0, wait_limit_us=20000)
    with pytest.raises(KrakenAmdError) as both:
        _waits.check(block=True)
    assert str(both.value).count("copy_engine_scatter") == 2
    assert time.perf_counter() - t0 < 0.1
    _waits.check(block=True)
    assert _waits.new_status(dev).item() == 0                             # cleared by the report
    # the all-gather matmul with chunks that never arrive (no copies are enqueued for this call)
    from kraken_amd.fused.all_gather_matmul import _matmul_w_progress
    m, K, Nn = 64, 128, 256
    a = orc.randn_bf16((4 * m, K), 1).to(dev)
    bT = orc.randn_bf16((Nn, K), 2, 0.05).to(dev)
    status = _waits.new_status(dev)
    _matmul_w_progress(a, a[:m], bT.T, torch.zeros(4, dtype=torch.int32, device=dev),
                       {"RANK": 0, "WORLD_SIZE": 4, "SPLITS_PER_RANK": 1, "wait_limit_us": 2000}, status)
    _waits.watch(status, "all_gather_matmul")
    with pytest.raises(KrakenAmdError, match="all_gather_matmul"):
        _waits.check(block=True)


def test_ce_persistent_reference_shape(dev):
    """(8192, 4096, 14336), the shape of test/test_gemm_reduce_scatter.py:93-111 (tolerance 1e-2
    there; the gate here is the library's 2e-2 on sampled rows)."""
    M, N, K, W, rank = 8192, 4096, 14336, 8, 5
    a = orc.randn_bf16((M, K), 42)
    b = orc.randn_bf16((N, K), 43, 0.02).T
    peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(W - 1)])
    out = fused.gemm_reduce_scatter_ce_persistent(a.to(dev), b.to(dev), peers=peers.to(dev), rank=rank)
    pick = torch.tensor([0, 1, 127, 128, 255, 256, 700, 1023])
    own = (a[rank * 1024 + pick].float() @ b.float()).to(BF16)
    bands = [p[pick] for p in peers]
    bands.insert(rank, own)
    want = orc.reduce_rotated(torch.cat(bands, 0), W, rank, acc_bf16=True)
    torch.testing.assert_close(out.cpu()[pick], want, **TOL)


def _sampled_rows_check(got, rows, a, b, extra, tol=TOL):
    want = a[rows].float() @ b.float()
    if extra is not None:
        want = want + extra
    torch.testing.assert_close(got.cpu()[rows].float(), want.to(BF16).float(), **tol)


def test_baseline_config4_full_size(dev, monkeypatch):
    """A [8192,3584] @ B [3584,8192]; band of 1024 rows + 7 partials.  Oracle on sampled rows."""
    monkeypatch.delenv("KRAKEN_AMD_GEMM_TILE", raising=False)
    monkeypatch.delenv("KRAKEN_AMD_GEMM_PEERS", raising=False)
    M, N, K, W, rank = 8192, 8192, 3584, 8, 3
    a = orc.randn_bf16((M, K), 42)
    b = orc.randn_bf16((K, N), 43, 0.02)
    peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(W - 1)])
    c_scratch = torch.empty(M, N, dtype=BF16, device=dev)
    out = fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=peers.to(dev), rank=rank, c_scratch=c_scratch)
    band = torch.arange(rank * 1024, (rank + 1) * 1024)
    pick = band[torch.tensor([0, 1, 31, 32, 255, 256, 511, 777, 1023])]
    want = a[pick].float() @ b.float() + peers[:, pick - rank * 1024].float().sum(0)
    torch.testing.assert_close(out.cpu()[pick - rank * 1024].float(), want.to(BF16).float(), **TOL)
    others = torch.tensor([0, 255, 256, 1023, 4096, 5000, 8191])
    _sampled_rows_check(c_scratch, others, a, b, None)
    # whole-matrix check against the device library GEMM in fp32
    ref = (a.to(dev).float() @ b.to(dev).float())
    ref_band = ref[band.to(dev)] + peers.to(dev).float().sum(0)
    torch.testing.assert_close(out.float(), ref_band.to(BF16).float(), **TOL)


def test_baseline_config5_full_size(dev, monkeypatch):
    monkeypatch.delenv("KRAKEN_AMD_GEMM_TILE", raising=False)
    monkeypatch.delenv("KRAKEN_AMD_GEMM_PEERS", raising=False)
    # fused all-reduce: A [4096,1024] @ B [1024,8192] + 7 partials + bias
    M, N, K, P = 4096, 8192, 1024, 7
    a = orc.randn_bf16((M, K), 42)
    b = orc.randn_bf16((K, N), 43, 0.02)
    peers = torch.stack([orc.randn_bf16((M, N), 100 + j) for j in range(P)])
    bias = orc.randn_bf16((N,), 42, 0.02)
    out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=peers.to(dev), bias=bias.to(dev),
                                               out_dtype=BF16)
    pick = torch.tensor([0, 63, 64, 127, 128, 2047, 4095])
    want = a[pick].float() @ b.float() + peers[:, pick].float().sum(0) + bias.float()
    torch.testing.assert_close(out.cpu()[pick].float(), want.to(BF16).float(), **TOL)
    ref = a.to(dev).float() @ b.to(dev).float() + peers.to(dev).float().sum(0) + bias.to(dev).float()
    torch.testing.assert_close(out.float(), ref.to(BF16).float(), **TOL)
    del peers, out, ref
    # all-gather matmul: A stack [8,1024,8192] @ B [8192,3584] (B.T contiguous)
    W, m, K2, N2 = 8, 1024, 8192, 3584
    stack = orc.make_stack(W, (m, K2), seed0=42)
    bT = orc.randn_bf16((N2, K2), 43, 0.02)
    ag, c = fused.all_gather_matmul(stack.to(dev), bT.to(dev).T, rank=5)
    assert torch.equal(ag.cpu(), stack.reshape(W * m, K2))
    rows = torch.tensor([0, 1023, 1024, 5 * 1024, 5 * 1024 + 17, 8191])
    _sampled_rows_check(c, rows, stack.reshape(W * m, K2), bT.T, None)
    ref = stack.to(dev).reshape(W * m, K2).float() @ bT.to(dev).T.float()
    torch.testing.assert_close(c.float(), ref.to(BF16).float(), **TOL)


def test_all_gather_matmul_reference_test_shape(dev, monkeypatch):
    """test/test_allgather_matmul.py:51-66: M=4096, N=6656, K=16384, bf16, B.T contiguous, here with W=8 shards of
    512 rows; the gathered A must be the exact stack, C within the gate of the sampled-row oracle
    and of the device's fp32 GEMM on the whole matrix."""
    monkeypatch.delenv("KRAKEN_AMD_GEMM_TILE", raising=False)
    monkeypatch.delenv("KRAKEN_AMD_GEMM_PEERS", raising=False)
    W, M, N, K = 8, 4096, 6656, 16384
    stack = orc.make_stack(W, (M // W, K), seed0=42)
    bT = orc.randn_bf16((N, K), 43, 0.02)
    sd = stack.to(dev)
    for rank in (0, 5):
        ag, c = fused.all_gather_matmul(sd, bT.to(dev).T, rank=rank)
        assert torch.equal(ag.cpu(), stack.reshape(M, K))
        rows = torch.tensor([0, 511, 512, 5 * 512 + 3, 4095])
        _sampled_rows_check(c, rows, stack.reshape(M, K), bT.T, None)
        ref = sd.reshape(M, K).float() @ bT.to(dev).T.float()
        torch.testing.assert_close(c.float(), ref.to(BF16).float(), **TOL)


@pytest.mark.parametrize("mode", ["mfma", "epilogue"])
def test_non_finite_partial_sum_stays_local(dev, monkeypatch, mode):
    """An Inf in one peer's partial sum: added in the epilogue it shows up in its own element
    only; added on the matrix cores (identity MFMA, 0 * Inf = NaN) it may also spoil the columns
    of its row that share its MFMA -- the aligned block of 32 -- and nothing else."""
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "256")
    monkeypatch.setenv("KRAKEN_AMD_GEMM_PEERS", mode)
    M, N, K, P = 512, 512, 256, 3
    a, b, peers = mk(M, N, K, P)
    r, c = 300, 77
    peers[1, r, c] = float("inf")
    out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=peers.to(dev), out_dtype=BF16).cpu().float()
    clean = peers.clone()
    clean[1, r, c] = 0.0
    want = orc.gemm_all_reduce(a, b, clean).to(BF16).float()
    bad = ~torch.isfinite(out)
    assert bad[r, c]
    group = torch.zeros_like(bad)
    group[r, c // 32 * 32:c // 32 * 32 + 32] = True
    assert not (bad & ~group).any()
    if mode == "epilogue":
        assert bad.sum() == 1 and out[r, c] == float("inf")
    torch.testing.assert_close(out[~group], want[~group], **TOL)


@pytest.mark.parametrize("P", [1, 2, 7, 8, 15])
def test_gemm_all_reduce_world_sizes(dev, tile, P):
    """Every world size the C ABI accepts (W = P + 1 up to 16), on a shape with whole-band
    256-tiles (matrix-core or epilogue peer path) and on a ragged one (generic epilogue path)."""
    for (M, N, K) in [(512, 256, 160), (200, 136, 72)]:
        a, b, peers = mk(M, N, K, P, seed=P)
        bias = orc.randn_bf16((N,), 9, 0.02)
        want = orc.gemm_all_reduce(a, b, peers, bias)
        out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=peers.to(dev), bias=bias.to(dev))
        torch.testing.assert_close(out.cpu(), want, rtol=1e-3, atol=1e-3)
        outb = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev), peers=peers.to(dev), bias=bias.to(dev),
                                                    out_dtype=BF16)
        torch.testing.assert_close(outb.cpu(), want.to(BF16), **TOL)


@pytest.mark.parametrize("P", [1, 3, 7, 15])
def test_separate_peer_buffers_match_the_stacked_form(dev, tile, P):
    """Pointer-table entry point: the peers' partial sums as P separate allocations give the
    stacked form's bits, on whole-band 256-tiles (matrix-core path, 7-peer and generic epilogue
    paths) and on a ragged shape."""
    for (M, N, K) in [(512, 512, 192), (200, 136, 72)]:
        a, b, peers = mk(M, N, K, P, seed=P)
        bias = orc.randn_bf16((N,), 9, 0.02)
        pads, plist = [], [None] * P
        for j in reversed(range(P)):
            pads.append(torch.empty(1208 * (j % 3 + 1), dtype=BF16, device=dev))
            plist[j] = peers[j].to(dev)
        ad, bd, pd, biasd = a.to(dev), b.to(dev), peers.to(dev), bias.to(dev)
        for dt in (torch.float32, BF16):
            o1 = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=biasd, out_dtype=dt)
            o2 = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=plist, bias=biasd, out_dtype=dt)
            assert torch.equal(o1, o2)
        torch.testing.assert_close(o2.cpu(), orc.gemm_all_reduce(a, b, peers, bias).to(BF16), **TOL)
    # reduce-scatter: band of rank 1 of W = P + 1, other bands to the scratch
    W = P + 1
    M, N, K = 256 * W, 256, 128
    a, b, _ = mk(M, N, K, 0)
    peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(P)])
    plist = [peers[j].to(dev) for j in range(P)]
    c1 = torch.zeros(M, N, dtype=BF16, device=dev)
    c2 = torch.zeros(M, N, dtype=BF16, device=dev)
    o1 = fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=peers.to(dev), rank=1, c_scratch=c1)
    o2 = fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=plist, rank=1, c_scratch=c2)
    assert torch.equal(o1, o2) and torch.equal(c1, c2)
    want, _ = orc.gemm_reduce_scatter(a, b, peers, 1, W)
    torch.testing.assert_close(o2.cpu(), want, **TOL)
    # the copy-engine variant takes a list as well
    o3 = fused.gemm_reduce_scatter_ce_persistent(a.to(dev), b.to(dev), peers=plist, rank=1, world_size=W)
    o4 = fused.gemm_reduce_scatter_ce_persistent(a.to(dev), b.to(dev), peers=peers.to(dev), rank=1, world_size=W)
    assert torch.equal(o3, o4)


@pytest.mark.parametrize("splits", [2, 3, 5, 16])
@pytest.mark.parametrize("b_t", [False, True])
def test_split_k_loop(dev, monkeypatch, splits, b_t):
    """Few output tiles: several workgroups share a tile's K loop, their partial products meet
    in the workspace.  Parity with the oracle for every epilogue form and the same bits run to
    run (the parts are summed in a fixed order)."""
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "128")
    monkeypatch.setenv("KRAKEN_AMD_GEMM_SPLITK", str(splits))
    for (M, N, K) in [(128, 384, 1024), (200, 136, 520), (256, 256, 64 * splits)]:
        a, b, peers = mk(M, N, K, 3, b_t, seed=splits)
        bias = orc.randn_bf16((N,), 42, 0.02)
        want = orc.gemm_all_reduce(a, b, peers, bias)
        ad, bd, pd, biasd = a.to(dev), b.to(dev), peers.to(dev), bias.to(dev)
        out = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=biasd)
        torch.testing.assert_close(out.cpu(), want, rtol=1e-3, atol=1e-3)
        for _ in range(3):
            again = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=biasd)
            assert torch.equal(out, again)
        outb = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=[p for p in pd], bias=biasd, out_dtype=BF16)
        torch.testing.assert_close(outb.cpu(), want.to(BF16), **TOL)
        plain = fused.gemm_one_shot_all_reduce_fused(ad, bd)
        torch.testing.assert_close(plain.cpu(), orc.gemm_all_reduce(a, b), rtol=1e-3, atol=1e-3)
    # reduce-scatter: band with peers, other bands to the scratch
    M, N, K, W = 512, 256, 640, 4
    a, b, _ = mk(M, N, K, 0, b_t)
    peers = torch.stack([orc.randn_bf16((M // W, N), 100 + j) for j in range(W - 1)])
    want, c_want = orc.gemm_reduce_scatter(a, b, peers, 2, W)
    c_scratch = torch.zeros(M, N, dtype=BF16, device=dev)
    out = fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=peers.to(dev), rank=2, c_scratch=c_scratch)
    torch.testing.assert_close(out.cpu(), want, **TOL)
    rows = torch.ones(M, dtype=torch.bool)
    rows[2 * M // W:3 * M // W] = False
    torch.testing.assert_close(c_scratch.cpu()[rows], c_want[rows], **TOL)


@pytest.mark.parametrize("b_t", [False, True])
@pytest.mark.parametrize("force", ["", "3"])
def test_tail_round_split(dev, monkeypatch, b_t, force):
    """272 tiles of 256 x 256 = one full round of 256 + 16: the 16 get several workgroups each
    (second launch) and a finishing pass; every epilogue form against the oracle, and the plain
    product against the one-launch result."""
    if force:
        monkeypatch.setenv("KRAKEN_AMD_GEMM_TAILSPLIT", force)
    M, N, K, W = 4352, 4096, 4096 if not force else 1024, 2
    assert _lib.load().kr_gemm_workspace_bytes(M, N, K) == 16 * (int(force) if force else 8) * 256 * 256 * 4
    a, b, _ = mk(M, N, K, 0, b_t, seed=5)
    ad, bd = a.to(dev), b.to(dev)
    prod = a.float() @ b.float()
    plain = fused.gemm_one_shot_all_reduce_fused(ad, bd)
    torch.testing.assert_close(plain.cpu(), prod, rtol=1e-3, atol=1e-3)
    assert torch.equal(plain, fused.gemm_one_shot_all_reduce_fused(ad, bd))          # reproducible
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TAILSPLIT", "0")
    one_launch = fused.gemm_one_shot_all_reduce_fused(ad, bd)
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TAILSPLIT", force) if force else monkeypatch.delenv("KRAKEN_AMD_GEMM_TAILSPLIT")
    torch.testing.assert_close(plain, one_launch, rtol=1e-4, atol=1e-4)
    assert not torch.equal(plain, one_launch) or K <= 64                              # the split did run
    # all-reduce form: peers and bias on every row, bf16 result
    peers = torch.stack([orc.randn_bf16((M, N), 100 + j) for j in range(2)])
    bias = orc.randn_bf16((N,), 9, 0.02)
    out = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=peers.to(dev), bias=bias.to(dev), out_dtype=BF16)
    want = (prod + peers.float().sum(0) + bias.float()).to(BF16)
    torch.testing.assert_close(out.cpu(), want, **TOL)
    # reduce-scatter form: band of rank 1 (rows 2176.., it starts inside a tile), other rows to the scratch
    rank = 1
    bp = torch.stack([orc.randn_bf16((M // W, N), 200 + j) for j in range(W - 1)])
    c_scratch = torch.zeros(M, N, dtype=BF16, device=dev)
    out = fused.gemm_reduce_scatter(ad, bd, peers=[p.to(dev) for p in bp], rank=rank, world_size=W, c_scratch=c_scratch)
    band = slice(rank * (M // W), (rank + 1) * (M // W))
    torch.testing.assert_close(out.cpu(), (prod[band] + bp.float().sum(0)).to(BF16), **TOL)
    rows = torch.ones(M, dtype=torch.bool)
    rows[band] = False
    torch.testing.assert_close(c_scratch.cpu()[rows], prod[rows].to(BF16), **TOL)


@pytest.mark.parametrize("b_t", [False, True])
def test_whole_launch_split_for_few_rows(dev, monkeypatch, b_t):
    """24 tiles of 256 x 256 and a long K loop: no full round at all, every tile's K loop is
    shared by 8 workgroups of the large-tile kernel.  Chosen by default for row-major B; forced
    for transposed-contiguous B (which takes this path only with more work per tile)."""
    M, N, K, W = 512, 3072, 8192, 4
    lib = _lib.load()
    if b_t:
        monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "256")
    assert lib.kr_gemm_workspace_bytes(M, N, K) == 24 * 8 * 256 * 256 * 4
    a, b, _ = mk(M, N, K, 0, b_t, seed=11)
    ad, bd = a.to(dev), b.to(dev)
    prod = a.float() @ b.float()
    plain = fused.gemm_one_shot_all_reduce_fused(ad, bd)
    torch.testing.assert_close(plain.cpu(), prod, rtol=1e-3, atol=2e-3)
    assert torch.equal(plain, fused.gemm_one_shot_all_reduce_fused(ad, bd))          # reproducible
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "128")
    other = fused.gemm_one_shot_all_reduce_fused(ad, bd)
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "256") if b_t else monkeypatch.delenv("KRAKEN_AMD_GEMM_TILE")
    torch.testing.assert_close(plain, other, rtol=1e-4, atol=1e-4)
    assert not torch.equal(plain, other)                                              # another kernel did run
    peers = torch.stack([orc.randn_bf16((M, N), 100 + j) for j in range(2)])
    bias = orc.randn_bf16((N,), 9, 0.02)
    out = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=peers.to(dev), bias=bias.to(dev), out_dtype=BF16)
    torch.testing.assert_close(out.cpu(), (prod + peers.float().sum(0) + bias.float()).to(BF16), **TOL)
    rank = 1                                     # band = rows 128..255, inside the first row of tiles
    bp = torch.stack([orc.randn_bf16((M // W, N), 200 + j) for j in range(W - 1)])
    c_scratch = torch.zeros(M, N, dtype=BF16, device=dev)
    out = fused.gemm_reduce_scatter(ad, bd, peers=bp.to(dev), rank=rank, world_size=W, c_scratch=c_scratch)
    band = slice(rank * (M // W), (rank + 1) * (M // W))
    torch.testing.assert_close(out.cpu(), (prod[band] + bp.float().sum(0)).to(BF16), **TOL)
    rows = torch.ones(M, dtype=torch.bool)
    rows[band] = False
    torch.testing.assert_close(c_scratch.cpu()[rows], prod[rows].to(BF16), **TOL)


@pytest.mark.parametrize("b_t", [False, True])
def test_ragged_shapes_on_the_large_tile(dev, monkeypatch, b_t):
    """M and N that 256 does not divide, on the 256 x 256 kernel: edge tiles read short operand
    panels and store through the bounds-checked epilogue; every epilogue form."""
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "256")
    for (M, N, K) in [(1000, 520, 192), (300, 264, 64), (513, 1032, 256), (768, 8, 128), (8, 768, 128)]:
        a, b, peers = mk(M, N, K, 2, b_t, seed=M)
        bias = orc.randn_bf16((N,), 42, 0.02)
        ad, bd, pd, biasd = a.to(dev), b.to(dev), peers.to(dev), bias.to(dev)
        want = orc.gemm_all_reduce(a, b, peers, bias)
        out = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=biasd)
        torch.testing.assert_close(out.cpu(), want, rtol=1e-3, atol=1e-3)
        outb = fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=biasd, out_dtype=BF16)
        torch.testing.assert_close(outb.cpu(), want.to(BF16), **TOL)
        plain = fused.gemm_one_shot_all_reduce_fused(ad, bd, out_dtype=BF16)
        torch.testing.assert_close(plain.cpu(), orc.gemm_all_reduce(a, b).to(BF16), **TOL)
    # reduce-scatter with a band that ends inside the ragged last tile; guard rows behind the outputs
    M, N, K, W = 1000, 520, 192, 4
    a, b, _ = mk(M, N, K, 0, b_t, seed=3)
    for rank in (0, 3):
        bp = torch.stack([orc.randn_bf16((M // W, N), 300 + j) for j in range(W - 1)])
        want, c_want = orc.gemm_reduce_scatter(a, b, bp, rank, W)
        c_scratch = torch.zeros(M + 8, N, dtype=BF16, device=dev)
        out = fused.gemm_reduce_scatter(a.to(dev), b.to(dev), peers=bp.to(dev), rank=rank, c_scratch=c_scratch[:M])
        torch.testing.assert_close(out.cpu(), want, **TOL)
        rows = torch.ones(M, dtype=torch.bool)
        rows[rank * (M // W):(rank + 1) * (M // W)] = False
        torch.testing.assert_close(c_scratch.cpu()[:M][rows], c_want[rows], **TOL)
        assert (c_scratch[M:] == 0).all()                     # nothing written past row M


def test_split_k_is_chosen_for_few_rows(dev):
    """The default heuristic: 128 x 6656 x 4096 (52 tiles) asks for a workspace, 4096 x 4096 does not."""
    lib = _lib.load()
    assert lib.kr_gemm_workspace_bytes(128, 6656, 4096) > 0
    assert lib.kr_gemm_workspace_bytes(4096, 4096, 4096) == 0
    assert lib.kr_gemm_workspace_bytes(128, 6656, 64) == 0          # one k-step: nothing to split
    a, b, _ = mk(128, 6656, 4096, 0, True)
    out = fused.gemm_one_shot_all_reduce_fused(a.to(dev), b.to(dev))
    torch.testing.assert_close(out.cpu(), orc.gemm_all_reduce(a, b), rtol=1e-3, atol=2e-3)


def test_gemm_paths_replay_from_a_graph(dev, monkeypatch):
    """The GEMM entry point enqueues kernels only (no allocation, no memset, no host sync), so a
    caller may capture it: three fused calls are captured once and replayed with eager work in
    between; every replay must reproduce the eager result bit for bit."""
    monkeypatch.delenv("KRAKEN_AMD_GEMM_TILE", raising=False)
    monkeypatch.delenv("KRAKEN_AMD_GEMM_PEERS", raising=False)
    M, N, K, W, rank = 1024, 512, 512, 4, 1
    a, b, peers_full = mk(M, N, K, W - 1)
    bias = orc.randn_bf16((N,), 3, 0.02)
    ad, bd, bias_d = a.to(dev), b.to(dev), bias.to(dev)
    bt = bd.T.contiguous().T               # all_gather_matmul wants b.T contiguous
    pf = peers_full.to(dev)
    pb = pf[:, :M // W].contiguous()
    eager = (fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pf, bias=bias_d, out_dtype=BF16),
             fused.gemm_reduce_scatter(ad, bd, peers=pb, rank=rank),
             fused.all_gather_matmul(ad.view(W, M // W, K), bt, rank=rank)[1])
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            got = (fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pf, bias=bias_d, out_dtype=BF16),
                   fused.gemm_reduce_scatter(ad, bd, peers=pb, rank=rank),
                   fused.all_gather_matmul(ad.view(W, M // W, K), bt, rank=rank)[1])
    for rep in range(3):
        for t in got:
            t.zero_()                      # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for e, r in zip(eager, got):
            assert torch.equal(e, r)


@pytest.mark.parametrize("peers_mode", ["epilogue", "mfma"])
@pytest.mark.parametrize("mfma", ["16", "32"])
def test_split_tiles_round_like_unsplit_tiles(dev, monkeypatch, peers_mode, mfma):
    """Tiles whose K loop is split (tail round, finished by a separate pass) and tiles of the main
    launch must round alike: with small-integer operands and peers and bias on a grid of 1/16
    every fp32 sum is exact whatever its order, so the split result has to equal the unsplit one
    bit for bit -- with peers and bias on a bf16 result, where rounding the product before or after
    the peers are added makes a visible difference."""
    M, N, K, P = 4352, 4096, 1024, 3          # 272 tiles of 256 x 256: 256 + 16 in the tail
    g = torch.Generator().manual_seed(5)
    a = torch.randint(-3, 4, (M, K), generator=g).to(BF16)
    b = torch.randint(-3, 4, (K, N), generator=g).to(BF16)
    peers = (torch.randint(-127, 128, (P, M, N), generator=g).float() / 16).to(BF16)
    bias = (torch.randint(-32, 33, (N,), generator=g).float() / 4).to(BF16)
    ad, bd, pd, biasd = a.to(dev), b.to(dev), peers.to(dev), bias.to(dev)
    monkeypatch.setenv("KRAKEN_AMD_GEMM_PEERS", peers_mode)
    monkeypatch.setenv("KRAKEN_AMD_GEMM_MFMA", mfma)
    res = {}
    for split in ("0", "3"):
        monkeypatch.setenv("KRAKEN_AMD_GEMM_TAILSPLIT", split)
        res[split] = [
            fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=biasd, out_dtype=BF16),
            fused.gemm_one_shot_all_reduce_fused(ad, bd, bias=biasd, out_dtype=BF16),
            fused.gemm_one_shot_all_reduce_fused(ad, bd, peers=pd, bias=biasd),
            fused.gemm_reduce_scatter(ad, bd, peers=pd[:1, : M // 2].contiguous(), rank=1, world_size=2),
        ]
    for x, y in zip(res["0"], res["3"]):
        assert torch.equal(x, y)
    # the exact product is large enough for the two rounding orders to differ somewhere
    prod = a.float() @ b.float()
    once = (prod + peers.float().sum(0) + bias.float()).to(BF16)
    twice = (prod.to(BF16).float() + peers.float().sum(0) + bias.float()).to(BF16)
    assert not torch.equal(once, twice)
