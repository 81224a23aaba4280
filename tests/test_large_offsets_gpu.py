"""Tensors of more than 2^31 elements (4 GiB of bf16): every kernel indexes with 64 bits.

The tensors are zero except for a few probed regions that straddle the byte offsets 2^31 and
2^32 and the two ends; the probed regions are compared with the oracle and the rest of the
output must stay zero (a wrapped index would land somewhere in it)."""
import pytest
import torch

from kraken_amd import comm, fused
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def same_bits(a, b):
    return torch.equal(a.cpu().contiguous().view(torch.int16), b.cpu().contiguous().view(torch.int16))


@pytest.mark.parametrize("as_list", [False, True])
def test_reduce_beyond_4_gib_per_buffer(dev, as_list):
    W, size = 2, 4096
    numel = (1 << 31) + (1 << 21)
    starts = [0, (1 << 30) - size // 2, (1 << 31) - size // 2, numel - size]
    stack = torch.zeros(W, numel, dtype=BF16, device=dev)
    patches = []
    for k, s in enumerate(starts):
        p = orc.make_stack(W, (size,), seed0=7 * k)
        stack[:, s:s + size] = p.to(dev)
        patches.append(p)
    bufs = [stack[0], stack[1].clone()] if as_list else stack
    out = comm.one_shot_all_reduce(bufs)
    assert out.shape == (numel,)
    nonzero = 0
    for s, p in zip(starts, patches):
        want = orc.reduce(p)
        assert same_bits(out[s:s + size], want), f"region at element {s}"
        nonzero += int(torch.count_nonzero(want))
    assert int(torch.count_nonzero(out)) == nonzero
    # the second rank's half of the same message (two-shot share): starts beyond 2^31 bytes
    share = comm.two_shot_all_reduce(bufs, rank=1)
    assert share.shape == (numel // 2,)
    assert torch.equal(share, out[numel // 2:])


def test_rms_norm_beyond_4_gib(dev):
    D = 8192
    rows = (1 << 18) + 8
    probe = [0, (1 << 17) - 1, 1 << 17, (1 << 18) - 1, 1 << 18, rows - 1]
    x = torch.zeros(rows, D, dtype=BF16, device=dev)
    xs = orc.randn_bf16((len(probe), D), 5)
    x[torch.tensor(probe, device=dev)] = xs.to(dev)
    w = orc.randn_bf16((D,), 6, 0.02) + 1
    y = fused.rms_norm(x, w.to(dev), 1e-5)
    want = orc.rms_norm(xs, w, 1e-5)
    got = y[torch.tensor(probe, device=dev)].cpu()
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    assert int(torch.count_nonzero(y)) == int(torch.count_nonzero(got))
    # reduce + bias + norm over two such buffers
    stack = torch.zeros(2, rows, D, dtype=BF16, device=dev)
    stack[0] = x
    stack[1, torch.tensor(probe, device=dev)] = xs.to(dev)
    y2 = torch.empty(rows, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias_rms_norm(stack, None, None, w.to(dev), y2)
    want2 = orc.rms_norm((2 * xs.float()).to(BF16), w, 1e-5)
    got2 = y2[torch.tensor(probe, device=dev)].cpu()
    torch.testing.assert_close(got2.float(), want2.float(), rtol=2e-2, atol=2e-2)
    assert int(torch.count_nonzero(y2)) == int(torch.count_nonzero(got2))


@pytest.mark.parametrize("tile", ["128", "256"])
def test_gemm_outputs_beyond_4_gib(dev, monkeypatch, tile):
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", tile)
    M, N, K, W = 65536 + 256, 32768, 256, 2
    a = orc.randn_bf16((M, K), 42).to(dev)
    b = orc.randn_bf16((K, N), 43, 0.05).to(dev)
    rows = torch.tensor([0, 32767, 32768, 32895, 32896, 65535, 65536, M - 1], device=dev)
    want = (a[rows].float() @ b.float()).to(BF16).float().cpu()
    out = fused.gemm_one_shot_all_reduce_fused(a, b, out_dtype=BF16)
    torch.testing.assert_close(out[rows].float().cpu(), want, rtol=2e-2, atol=2e-2)
    del out
    # reduce-scatter form: rank 1's band (rows 32896..) to the result, rank 0's rows to the scratch
    c_scratch = torch.zeros(M, N, dtype=BF16, device=dev)
    peers = torch.zeros(1, M // W, N, dtype=BF16, device=dev)
    peers[0, M // W - 1] = 1.0
    band = fused.gemm_reduce_scatter(a, b, peers=peers, rank=1, world_size=W, c_scratch=c_scratch)
    lo = rows[rows < M // W]
    hi = rows[rows >= M // W]
    torch.testing.assert_close(c_scratch[lo].float().cpu(), want[: len(lo)], rtol=2e-2, atol=2e-2)
    extra = torch.zeros(len(hi), 1)
    extra[-1] = 1.0                      # the last row of the band got the peer's 1.0
    torch.testing.assert_close(band[hi - M // W].float().cpu(), (want[len(lo):] + extra).to(BF16).float(),
                               rtol=2e-2, atol=2e-2)
    assert int(torch.count_nonzero(c_scratch[M // W:])) == 0        # the band never goes to the scratch
