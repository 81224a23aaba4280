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


_FRESH = r"""
import sys, torch
sys.path.insert(0, {root!r})
from kraken_amd import _lib
from oracle import oracle as orc
dev = torch.device("cuda:0")
lib = _lib.load()
M, N, K = 128, 6656, 4096
need = lib.kr_gemm_workspace_bytes(M, N, K)
assert 0 < need <= (64 << 20)
a = orc.randn_bf16((M, K), 1).to(dev); b = orc.randn_bf16((K, N), 2, 0.05).to(dev)
got = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
want = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
ws = torch.empty(need, dtype=torch.uint8, device=dev)
torch.cuda.synchronize()
stream = torch.cuda.current_stream(dev).cuda_stream
args = lambda out: [a.data_ptr(), K, 1, b.data_ptr(), N, 1, M, N, K, None, 0, 0, None, 0, M, None, out.data_ptr(), 0, 0]
if {init}:
    assert lib.kr_init() == 0
    torch.cuda.synchronize()
free_before, _ = torch.cuda.mem_get_info(dev)
# the entry point under test is the first kernel launch of this library in the process
rc = lib.kr_gemm_reduce_noalloc_bf16(*args(got), stream)
assert rc == 0, rc
torch.cuda.synchronize()
free_after, _ = torch.cuda.mem_get_info(dev)
if {init}:
    assert free_after == free_before, (free_before, free_after)
assert lib.kr_gemm_reduce_ws_bf16(*args(want), ws.data_ptr(), need, stream) == 0
torch.cuda.synchronize()
assert torch.equal(got, want)
print("fresh-process ok", free_before - free_after)
"""


@pytest.mark.parametrize("init", [True, False])
def test_first_call_in_a_fresh_process(init):
    """The entry point as the very first launch of the library in a process: after kr_init() the
    call moves no device memory (the code object and its scratch array are already resident);
    without kr_init() it still gives the bits of the workspace form."""
    import subprocess
    import sys
    from pathlib import Path

    root = str(Path(__file__).resolve().parent.parent)
    out = subprocess.run([sys.executable, "-c", _FRESH.format(root=root, init=init)], capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "fresh-process ok" in out.stdout


def test_captured_in_a_graph_and_replayed(dev):
    """A split-shape call captured into a HIP graph after kr_init(): every replay gives the bits of
    the workspace form, with eager work of the same entry point (another shape, same scratch array)
    between the replays."""
    lib = _lib.load()
    assert lib.kr_init() == 0
    M, N, K = 128, 6656, 4096
    need = lib.kr_gemm_workspace_bytes(M, N, K)
    a, b, peers, bias, ad, bd, pd, biasd = _operands(M, N, K, 2, 11, dev)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    want = torch.empty(M, N, dtype=BF16, device=dev)
    got = torch.zeros(M, N, dtype=BF16, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    assert lib.kr_gemm_reduce_ws_bf16(*_args(ad, bd, pd, biasd, want, M, N, K), ws.data_ptr(), need, stream) == 0
    # the eager call between the replays: a smaller split shape that overwrites part of the array
    M2, N2, K2 = 128, 1024, 2048
    a2, b2, peers2, bias2, ad2, bd2, pd2, biasd2 = _operands(M2, N2, K2, 2, 12, dev)
    got2 = torch.zeros(M2, N2, dtype=BF16, device=dev)
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.kr_gemm_reduce_noalloc_bf16(*_args(ad, bd, pd, biasd, got, M, N, K),
                                                 torch.cuda.current_stream(dev).cuda_stream)
            assert rc == 0, _lib.strerror(rc)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for replay in range(3):
        got.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), replay
        assert lib.kr_gemm_reduce_noalloc_bf16(*_args(ad2, bd2, pd2, biasd2, got2, M2, N2, K2), stream) == 0
        torch.cuda.synchronize()
