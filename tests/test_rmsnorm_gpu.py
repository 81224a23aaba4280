"""GPU parity of reduce+bias+RMSNorm and stand-alone RMSNorm against the CPU oracle.
Gate: rtol = atol = 2e-2 (bf16 output vs fp32-accumulated reference); additionally the
results must be within one bf16 ulp of the oracle (only the fp32 order of the sum of
squares and the rsqrt approximation differ)."""
import pytest
import torch

from kraken_amd import fused
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
TOL = dict(rtol=2e-2, atol=2e-2)


def assert_one_ulp(got, want):
    g, w = got.cpu().float(), want.float()
    d = (g - w).abs()
    assert (d <= w.abs() * 2.0 ** -7 + 1e-30).all(), float(d.max())
    assert (d == 0).float().mean() > 0.97


@pytest.mark.parametrize("D", [8, 64, 320, 2048, 4096, 5120, 8192, 16384, 65536])
@pytest.mark.parametrize("rows", [1, 5])
def test_rms_norm_row_lengths(dev, D, rows):
    x = orc.randn_bf16((rows, D), 3)
    w = orc.randn_bf16((D,), 4)
    y = fused.rms_norm(x.to(dev), w.to(dev), 1e-5)
    want = orc.rms_norm(x, w, 1e-5)
    torch.testing.assert_close(y.cpu(), want, **TOL)
    assert_one_ulp(y, want)


def test_rms_norm_closed_forms(dev):
    D = 1024
    w = orc.randn_bf16((D,), 6, 0.02, 1.0)
    x = torch.full((3, D), 3.0, dtype=BF16)
    y = fused.rms_norm(x.to(dev), w.to(dev), 1e-5).cpu()
    want = (w.float() * (3.0 / (9.0 + 1e-5) ** 0.5)).to(BF16)
    assert_one_ulp(y[1], want)
    z = fused.rms_norm(torch.zeros(3, D, dtype=BF16, device=dev), w.to(dev)).cpu()
    assert torch.equal(z, torch.zeros(3, D, dtype=BF16))
    yy = fused.rms_norm(orc.randn_bf16((4, D), 8).to(dev), torch.ones(D, dtype=BF16, device=dev)).float()
    torch.testing.assert_close((yy * yy).mean(-1).cpu(), torch.ones(4), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("b", [1, 2, 4, 8, 16, 32, 64])
def test_reference_test_shapes(dev, b):
    # test/test_allreduce_bias_rms_norm.py:56-86: x [b,5120] seed 42+rank+b, bias [b,5120] and
    # w [5120] seed 42+b, buffer (1024,1024); golden = all_reduce -> +bias -> rms_norm; tol 4e-2
    W = 8
    xs = [orc.randn_bf16((b, 5120), 42 + r + b) for r in range(W)]
    bias = orc.randn_bf16((b, 5120), 42 + b)
    w = orc.randn_bf16((5120,), 4242 + b)
    buf = torch.zeros(W, 1024, 1024, dtype=BF16, device=dev)
    for r in range(1, W):
        buf[r].view(-1)[: b * 5120].copy_(xs[r].view(-1))
    for fn in (fused.one_shot_all_reduce_bias_rms_norm, fused.two_shot_all_reduce_bias_rms_norm):
        y = torch.empty(b, 5120, dtype=BF16, device=dev)
        fn(buf, xs[0].to(dev), bias.to(dev), w.to(dev), y)
        want = orc.reduce_bias_rms_norm(torch.stack(xs), bias, w)
        torch.testing.assert_close(y.cpu(), want, **TOL)
        assert_one_ulp(y, want)
        # the reference's own golden: rms_norm of the bf16-rounded all-reduce + bias
        golden = orc.rms_norm((orc.reduce_library(torch.stack(xs)) + bias), w)
        torch.testing.assert_close(y.cpu(), golden, rtol=4e-2, atol=4e-2)


@pytest.mark.parametrize("W", [1, 2, 3, 4, 8, 16])
@pytest.mark.parametrize("bias_mode", ["none", "full", "vector"])
def test_world_sizes_and_bias_modes(dev, W, bias_mode):
    rows, D = 9, 1000
    stack = orc.make_stack(W, (rows, D))
    w = orc.randn_bf16((D,), 5, 0.02, 1.0)
    bias = {"none": None, "full": orc.randn_bf16((rows, D), 7), "vector": orc.randn_bf16((D,), 7, 0.02)}[bias_mode]
    y = torch.empty(rows, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias_rms_norm(stack.to(dev), None, None if bias is None else bias.to(dev),
                                            w.to(dev), y, eps=1e-5)
    want = orc.reduce_bias_rms_norm(stack, bias, w, 1e-5)
    torch.testing.assert_close(y.cpu(), want, **TOL)
    assert_one_ulp(y, want)


@pytest.mark.parametrize("W,rows,D", [(1, 3, 64), (3, 9, 1000), (8, 16, 8192), (8, 5, 16384), (16, 2, 65536)])
def test_separate_buffers_match_the_stacked_form(dev, W, rows, D):
    """Pointer-table entry point: W separate allocations give exactly the stacked form's bits
    (same kernel), for the short-row, grouped and long-row code paths."""
    stack = orc.make_stack(W, (rows, D), seed0=21)
    w = orc.randn_bf16((D,), 5, 0.02, 1.0)
    pads, bufs = [], [None] * W
    for r in reversed(range(W)):
        pads.append(torch.empty(808 * (r % 3 + 1), dtype=BF16, device=dev))
        bufs[r] = stack[r].to(dev)
    sd = stack.to(dev)
    for bias in (None, orc.randn_bf16((rows, D), 7), orc.randn_bf16((D,), 7, 0.02)):
        bd = None if bias is None else bias.to(dev)
        y1 = torch.empty(rows, D, dtype=BF16, device=dev)
        y2 = torch.empty(rows, D, dtype=BF16, device=dev)
        fused.one_shot_all_reduce_bias_rms_norm(sd, None, bd, w.to(dev), y1, eps=1e-5)
        fused.one_shot_all_reduce_bias_rms_norm(bufs, None, bd, w.to(dev), y2, eps=1e-5)
        assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
        assert_one_ulp(y2, orc.reduce_bias_rms_norm(stack, bias, w, 1e-5))
    if (rows * D) % (W * 16) == 0 and D % W == 0:
        y3 = torch.empty(rows, D, dtype=BF16, device=dev)
        x = orc.randn_bf16((rows, D), 31)
        fused.two_shot_all_reduce_bias_rms_norm(bufs, x.to(dev), None, w.to(dev), y3, rank=0)
        staged = stack.clone()
        staged[0] = x
        assert_one_ulp(y3, orc.reduce_bias_rms_norm(staged, None, w, 1e-5))


def test_nd_input_and_eps(dev):
    W, B, T, D = 4, 3, 5, 512
    stack = orc.make_stack(W, (B, T, D))
    bias, w = orc.make_bias_weight(D)
    y = torch.empty(B, T, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias_rms_norm(stack.to(dev), None, bias.to(dev), w.to(dev), y, eps=1e-2)
    assert_one_ulp(y, orc.reduce_bias_rms_norm(stack, bias, w, 1e-2))


@pytest.mark.parametrize("cfg", [(8, 256, 4096), (8, 16, 8192)])
def test_baseline_configs_1_and_3(dev, cfg):
    W, rows, D = cfg
    stack = orc.make_stack(W, (rows, D), seed0=42)
    bias, w = orc.make_bias_weight(D, 42)
    y = torch.empty(rows, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias_rms_norm(stack.to(dev), None, bias.to(dev), w.to(dev), y, eps=1e-5)
    want = orc.reduce_bias_rms_norm(stack, bias, w, 1e-5)
    torch.testing.assert_close(y.cpu(), want, **TOL)
    assert_one_ulp(y, want)
    torch.testing.assert_close(y.cpu(), orc.reduce_bias_rms_norm_library(stack, bias, w, 1e-5), **TOL)
    # scale invariance: x -> 2x (exact in bf16) changes nothing while mean(s^2) >> eps
    y2 = torch.empty_like(y)
    fused.one_shot_all_reduce_bias_rms_norm((stack * 2).to(dev), None, (bias * 2).to(dev), w.to(dev), y2, eps=1e-5)
    torch.testing.assert_close(y2.float().cpu(), y.float().cpu(), rtol=2 ** -7, atol=1e-5)


# ---- a few long rows: one row spread over many compute units (split-row kernel) ----------------

def _split_used(W, rows, D):
    from kraken_amd import _lib
    return _lib.load().kr_rmsnorm_workspace_bytes(W, rows, D) > 0


@pytest.mark.parametrize("W,rows,D", [(8, 16, 8192), (8, 1, 8192), (8, 5, 16384), (4, 3, 32768), (8, 7, 8200),
                                      (2, 3, 1024), (1, 2, 4096), (8, 64, 1024)])
@pytest.mark.parametrize("bias_mode", ["none", "full", "vector"])
def test_split_rows_match_the_oracle(dev, monkeypatch, W, rows, D, bias_mode):
    """Forced on for every shape it can take: rows whose last wavefront is ragged (D = 8200),
    two to 64 wavefronts per row, every W it is instantiated for, every bias form; stacked and
    separate buffers give the same bits; against the one-workgroup kernel at most an ulp."""
    monkeypatch.setenv("KRAKEN_AMD_ROW_SPLIT", "1")
    assert _split_used(W, rows, D)
    stack = orc.make_stack(W, (rows, D), seed0=11)
    w = orc.randn_bf16((D,), 5, 0.02, 1.0)
    bias = {"none": None, "full": orc.randn_bf16((rows, D), 7), "vector": orc.randn_bf16((D,), 7, 0.02)}[bias_mode]
    bd = None if bias is None else bias.to(dev)
    sd, wd = stack.to(dev), w.to(dev)
    want = orc.reduce_bias_rms_norm(stack, bias, w, 1e-5)
    y = torch.empty(rows, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias_rms_norm(sd, None, bd, wd, y, eps=1e-5)
    torch.testing.assert_close(y.cpu(), want, **TOL)
    assert_one_ulp(y, want)
    y2 = torch.full_like(y, 3.0)
    fused.one_shot_all_reduce_bias_rms_norm([sd[r].clone() for r in range(W)], None, bd, wd, y2, eps=1e-5)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))
    monkeypatch.setenv("KRAKEN_AMD_ROW_SPLIT", "0")
    assert not _split_used(W, rows, D)
    y3 = torch.empty_like(y)
    fused.one_shot_all_reduce_bias_rms_norm(sd, None, bd, wd, y3, eps=1e-5)
    assert_one_ulp(y3, want)
    assert (y3 == y).float().mean() > 0.99


def test_split_rows_default_rule(dev):
    """The decode shape of the benchmark takes the split kernel by default, the 256-row shape and
    short rows do not."""
    assert _split_used(8, 16, 8192) and _split_used(8, 1, 8192)
    assert not _split_used(8, 256, 4096) and not _split_used(8, 16, 1024) and not _split_used(3, 16, 8192)


def test_split_rows_share_one_workspace_across_shapes_and_calls(dev, monkeypatch):
    """Calls of different shapes in a row on one stream share the stream's workspace, which is never
    cleared in between: slots left by a wider call must not be taken for this call's."""
    monkeypatch.setenv("KRAKEN_AMD_ROW_SPLIT", "1")
    cases = []
    for i, (W, rows, D) in enumerate([(8, 16, 8192), (8, 3, 32768), (4, 64, 1024), (8, 1, 8192), (2, 16, 16384)]):
        stack = orc.make_stack(W, (rows, D), seed0=50 + i)
        bias, w = orc.make_bias_weight(D, 60 + i)
        cases.append((stack.to(dev), bias.to(dev), w.to(dev), torch.empty(rows, D, dtype=BF16, device=dev),
                      orc.reduce_bias_rms_norm(stack, bias, w, 1e-5)))
    for rep in range(4):
        order = cases if rep % 2 == 0 else cases[::-1]
        for (sd, bd, wd, y, want) in order:
            y.zero_()
            fused.one_shot_all_reduce_bias_rms_norm(sd, None, bd, wd, y, eps=1e-5)
        torch.cuda.synchronize()
        for (sd, bd, wd, y, want) in cases:
            assert_one_ulp(y, want)


def test_split_rows_replay_from_a_graph(dev):
    """Captured once, replayed with eager calls on the capture stream in between (they use the
    workspace the graph has baked in and advance its rows' generations): every replay gives the
    eager bits."""
    W, rows, D = 8, 16, 8192
    assert _split_used(W, rows, D)
    stack = orc.make_stack(W, (rows, D), seed0=42).to(dev)
    bias, w = (t.to(dev) for t in orc.make_bias_weight(D, 42))
    y = torch.empty(rows, D, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias_rms_norm(stack, None, bias, w, y)
    eager = y.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    yg = torch.empty_like(y)
    with torch.cuda.stream(side):
        fused.one_shot_all_reduce_bias_rms_norm(stack, None, bias, w, yg)   # the stream's workspace exists
        side.synchronize()
        with torch.cuda.graph(g, stream=side):
            for _ in range(3):
                fused.one_shot_all_reduce_bias_rms_norm(stack, None, bias, w, yg)
    for rep in range(3):
        yg.zero_()
        y.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):                                              # eager work between the replays,
            fused.one_shot_all_reduce_bias_rms_norm(stack, None, bias, w, y)       # on the graph's workspace
        torch.cuda.synchronize()
        assert torch.equal(y, eager)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(yg, eager)


def test_split_rows_report_through_the_status_word(dev):
    """The exchange of a row's wavefronts is a bounded wait like the flag waits: the wrapper hands the
    kernel the stream's status word and registers it (rate-limited); a normal call leaves it at zero
    and check(block=True) has nothing to raise."""
    from kraken_amd import _waits
    W, rows, D = 8, 16, 8192
    assert _split_used(W, rows, D)
    stack = orc.make_stack(W, (rows, D), seed0=3).to(dev)
    bias, w = (t.to(dev) for t in orc.make_bias_weight(D, 3))
    y = torch.empty(rows, D, dtype=BF16, device=dev)
    _waits.check(block=True)
    for _ in range(20):
        fused.one_shot_all_reduce_bias_rms_norm(stack, None, bias, w, y)
    assert _waits.new_status(dev).item() == 0
    _waits.check(block=True)
    assert len(_waits._pending) == 0
