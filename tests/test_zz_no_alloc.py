"""kr_gemm_reduce_noalloc_bf16: the split-K GEMM whose workspace is the library's own device
array, for callers that cannot allocate.  Through the C ABI it must give the bits of
kr_gemm_reduce_ws_bf16 with a caller-allocated workspace -- on two calls in a row, the second
on a smaller input (the array keeps the first call's contents) -- and must itself allocate
nothing."""
import pytest
import torch

from kraken_amd import _lib
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _operands(M, N, K, P, seed, dev):
    a = orc.randn_bf16((M, K), 42 + seed)
    b = orc.randn_bf16((K, N), 43 + seed, 0.05)
    peers = torch.stack([orc.randn_bf16((M, N), 100 + seed + j) for j in range(P)])
    bias = orc.randn_bf16((N,), 7 + seed, 0.02)
    return a, b, peers, bias, a.to(dev), b.to(dev), peers.to(dev), bias.to(dev)


def _args(ad, bd, pd, biasd, out, M, N, K):
    return [ad.data_ptr(), K, 1, bd.data_ptr(), N, 1, M, N, K, pd.data_ptr(), pd.shape[0], M * N,
            biasd.data_ptr(), 0, M, None, out.data_ptr(), 0, 0]


# (M, N, K): a few tiles of the 128x128 kernel whose K loop is split; one full round of 256x256
# tiles plus 16 tail tiles with 8 workgroups each; then smaller shapes of both kinds
SHAPES = [(128, 6656, 4096), (4352, 4096, 4096), (128, 1024, 2048), (512, 3072, 8192), (128, 384, 1024)]


def test_static_scratch_matches_caller_workspace(dev):
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    cases = []
    for i, (M, N, K) in enumerate(SHAPES):
        need = lib.kr_gemm_workspace_bytes(M, N, K)
        assert 0 < need <= (64 << 20), (M, N, K, need)
        a, b, peers, bias, ad, bd, pd, biasd = _operands(M, N, K, 2, i, dev)
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        want = torch.empty(M, N, dtype=BF16, device=dev)
        rc = lib.kr_gemm_reduce_ws_bf16(*_args(ad, bd, pd, biasd, want, M, N, K), ws.data_ptr(), need, stream)
        assert rc == 0, _lib.strerror(rc)
        got = torch.zeros(M, N, dtype=BF16, device=dev)
        cases.append((M, N, K, a, b, peers, bias, ad, bd, pd, biasd, want, got))
    torch.cuda.synchronize()

    # the calls under test, back to back on one stream, large then small, with nothing between
    # them: no allocation may happen (torch's allocator is not involved, and the device's free
    # memory must not move)
    free_before, _ = torch.cuda.mem_get_info(dev)
    for (M, N, K, a, b, peers, bias, ad, bd, pd, biasd, want, got) in cases:
        rc = lib.kr_gemm_reduce_noalloc_bf16(*_args(ad, bd, pd, biasd, got, M, N, K), stream)
        assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before

    for (M, N, K, a, b, peers, bias, ad, bd, pd, biasd, want, got) in cases:
        assert torch.equal(got, want), (M, N, K)
        rows = torch.tensor([0, M // 2, M - 1])
        ref = (a[rows].float() @ b.float() + peers[:, rows].float().sum(0) + bias.float()).to(BF16)
        torch.testing.assert_close(got.cpu()[rows], ref, rtol=2e-2, atol=2e-2)

    # once more in the opposite order (small first), same bits
    for (M, N, K, a, b, peers, bias, ad, bd, pd, biasd, want, got) in reversed(cases):
        got.zero_()
        rc = lib.kr_gemm_reduce_noalloc_bf16(*_args(ad, bd, pd, biasd, got, M, N, K), stream)
        assert rc == 0, _lib.strerror(rc)
    torch.cuda.synchronize()
    for (M, N, K, *_, want, got) in cases:
        assert torch.equal(got, want), (M, N, K)


def test_unsplit_shape_and_oversize(dev):
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    # a shape that is not split uses no scratch and equals the plain entry point
    M, N, K = 256, 256, 64
    assert lib.kr_gemm_workspace_bytes(M, N, K) == 0
    a, b, peers, bias, ad, bd, pd, biasd = _operands(M, N, K, 1, 3, dev)
    want = torch.empty(M, N, dtype=BF16, device=dev)
    got = torch.empty(M, N, dtype=BF16, device=dev)
    assert lib.kr_gemm_reduce_bf16(*_args(ad, bd, pd, biasd, want, M, N, K), stream) == 0
    assert lib.kr_gemm_reduce_noalloc_bf16(*_args(ad, bd, pd, biasd, got, M, N, K), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
