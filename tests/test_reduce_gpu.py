"""GPU parity of the W-way reduce (+bias) paths against the CPU oracle: bit-exact
(fp32 sums in a fixed order, one round-to-nearest-even)."""
import pytest
import torch

from kraken_amd import comm, fused
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def same_bits(a, b):
    return torch.equal(a.cpu().contiguous().view(torch.int16), b.cpu().contiguous().view(torch.int16))


@pytest.mark.parametrize("W", [1, 2, 3, 4, 5, 8, 16])
@pytest.mark.parametrize("shape", [(8,), (3, 8), (513, 24), (64, 5120), (1024, 1024)])
def test_one_shot_all_reduce_bit_exact(dev, W, shape):
    stack = orc.make_stack(W, shape)
    out = comm.one_shot_all_reduce(stack.to(dev))
    assert out.shape == stack.shape[1:] and out.dtype == BF16
    assert same_bits(out, orc.reduce(stack))


def test_one_shot_all_reduce_reference_test_tolerance(dev):
    # test/test_allreduce.py:48-66: bf16 [1024,1024], seed 42+rank, rtol=atol=1e-1 vs all_reduce
    W = 4
    stack = orc.make_stack(W, (1024, 1024), seed0=42)
    out = comm.one_shot_all_reduce(stack.to(dev)).cpu()
    torch.testing.assert_close(out, orc.reduce_library(stack), rtol=1e-1, atol=1e-1)
    torch.testing.assert_close(out.float(), stack.float().sum(0), rtol=2e-2, atol=2e-2)


def test_closed_form_rank_multiples(dev):
    W, c = 8, 0.25
    stack = torch.stack([torch.full((16, 64), (r + 1) * c, dtype=BF16) for r in range(W)])
    out = comm.one_shot_all_reduce(stack.to(dev)).cpu()
    assert torch.equal(out.float(), torch.full((16, 64), c * W * (W + 1) / 2))


@pytest.mark.parametrize("b", [1, 2, 4, 8, 16, 32, 64])
@pytest.mark.parametrize("W", [4, 8])
def test_one_shot_bias_reference_shapes(dev, b, W):
    # test/test_allreduce_bias.py:53-79: x [b,5120] seed 42+rank+b, bias [b,5120] seed 42+b,
    # symmetric buffer (1024,1024) larger than the message, tolerance 5e-2
    xs = [orc.randn_bf16((b, 5120), 42 + r + b) for r in range(W)]
    bias = orc.randn_bf16((b, 5120), 42 + b)
    buf = torch.zeros(W, 1024, 1024, dtype=BF16, device=dev)
    for r in range(1, W):
        buf[r].view(-1)[: b * 5120].copy_(xs[r].view(-1))
    out = torch.empty(b, 5120, dtype=BF16, device=dev)
    fused.one_shot_all_reduce_bias(buf, xs[0].to(dev), bias.to(dev), out, rank=0)   # copy-in of rank 0
    want = orc.reduce(torch.stack(xs), bias, bias_first=True)
    assert same_bits(out, want)
    torch.testing.assert_close(out.cpu(), orc.reduce_library(torch.stack(xs), bias), rtol=5e-2, atol=5e-2)
    # two-shot order (bias last), full result
    out2 = torch.empty(b, 5120, dtype=BF16, device=dev)
    ret = fused.two_shot_all_reduce_bias(buf, xs[0].to(dev), bias.to(dev), out2, rank=0)
    assert ret is out2
    assert same_bits(out2, orc.reduce(torch.stack(xs), bias, bias_first=False))


@pytest.mark.parametrize("bias_mode", ["none", "full", "vector"])
@pytest.mark.parametrize("bias_first", [True, False])
@pytest.mark.parametrize("W", [2, 3, 8])
def test_bias_modes_and_orders(dev, bias_mode, bias_first, W):
    rows, D = 37, 264          # ragged: 37*264/8 = 1221 vectors
    stack = orc.make_stack(W, (rows, D))
    bias = {"none": None, "full": orc.randn_bf16((rows, D), 7), "vector": orc.randn_bf16((D,), 7)}[bias_mode]
    out = torch.empty(rows, D, dtype=BF16, device=dev)
    bd = None if bias is None else bias.to(dev)
    if bias_first:
        fused.one_shot_all_reduce_bias(stack.to(dev), None, bd, out)
    else:
        fused.two_shot_all_reduce_bias(stack.to(dev), None, bd, out, BLOCK_SIZE=128 * W)
    assert same_bits(out, orc.reduce(stack, bias, bias_first))


def test_negative_zero_and_specials(dev):
    W = 4
    stack = torch.zeros(W, 16, dtype=BF16)
    stack[:, 0] = -0.0
    stack[0, 1], stack[1, 1] = float("inf"), 1.0
    stack[0, 2], stack[1, 2] = float("inf"), float("-inf")
    stack[0, 3] = 3.0e38
    stack[1, 3] = 3.0e38                                   # overflows fp32? no: 6e38 > fp32 max -> inf
    out = comm.one_shot_all_reduce(stack.to(dev)).cpu()
    want = orc.reduce(stack)
    assert torch.equal(torch.isnan(out), torch.isnan(want))
    ok = ~torch.isnan(want)
    assert same_bits(out[ok], want[ok])


def scattered(stack, dev):
    """The W slices of a host stack as W separate device allocations, irregularly spaced and in
    no address order (what a table of real peer mappings looks like)."""
    W = stack.shape[0]
    bufs, pads = [None] * W, []
    for r in reversed(range(W)):
        pads.append(torch.empty(1000 * (r % 3 + 1) + 8, dtype=BF16, device=dev))   # irregular gaps
        bufs[r] = stack[r].to(dev)
    return bufs


@pytest.mark.parametrize("W", [1, 2, 3, 8, 16])
def test_separate_buffers_match_the_stacked_form(dev, W):
    """Pointer-table entry points: W separate allocations give the oracle's bits, i.e. the
    same as the stacked form, for every reduce wrapper."""
    rows, D = 45, 264
    stack = orc.make_stack(W, (rows, D), seed0=11)
    bufs = scattered(stack, dev)
    assert same_bits(comm.one_shot_all_reduce(bufs), orc.reduce(stack))
    assert same_bits(comm.two_shot_all_reduce(bufs, rank=None, BLOCK_SIZE=128 * W), orc.reduce(stack))
    full_bias, vec_bias = orc.randn_bf16((rows, D), 7), orc.randn_bf16((D,), 8)
    out = torch.empty(rows, D, dtype=BF16, device=dev)
    for bias in (None, full_bias, vec_bias):
        bd = None if bias is None else bias.to(dev)
        fused.one_shot_all_reduce_bias(bufs, None, bd, out)
        assert same_bits(out, orc.reduce(stack, bias, bias_first=True))
        fused.two_shot_all_reduce_bias(bufs, None, bd, out, BLOCK_SIZE=128 * W)
        assert same_bits(out, orc.reduce(stack, bias, bias_first=False))
    # copy-in of this rank's input into its own buffer of the list
    x = orc.randn_bf16((rows, D), 99)
    rank = W - 1
    fused.one_shot_all_reduce_bias(bufs, x.to(dev), full_bias.to(dev), out, rank=rank)
    staged = stack.clone()
    staged[rank] = x
    assert same_bits(out, orc.reduce(staged, full_bias, bias_first=True))


def test_separate_buffers_two_shot_shares(dev):
    W, numel, block = 8, 2048 * 8 * 3 + 8 * 100, 2048
    stack = orc.make_stack(W, (numel,), seed0=5)
    bufs = scattered(stack, dev)
    bias = orc.randn_bf16((numel,), 9)
    full = orc.reduce(stack, bias, bias_first=False)
    assembled = torch.empty_like(full)
    for rank in range(W):
        idx = orc.striped_indices(numel, W, block, rank)
        share = comm.two_shot_all_reduce(bufs, rank=rank, layout="striped", BLOCK_SIZE=block)
        assert same_bits(share, orc.reduce_striped(stack, None, block, rank))
        out = torch.empty(idx.numel(), dtype=BF16, device=dev)
        fused.two_shot_all_reduce_bias(bufs, None, bias.to(dev), out, BLOCK_SIZE=block, rank=rank,
                                       layout="striped", numel=numel)
        assembled[idx] = out.cpu()
    assert same_bits(assembled, full)
    # contiguous shares: every entry of the table is moved on by the share's offset
    stack2 = orc.make_stack(W, (64, 256), seed0=6)
    bufs2 = scattered(stack2, dev)
    for rank in (0, 5, 7):
        share = comm.two_shot_all_reduce(bufs2, rank=rank)
        assert share.shape == (8, 256)
        assert same_bits(share, orc.reduce(stack2[:, rank * 8:(rank + 1) * 8]))


def test_separate_buffers_full_size_config2(dev):
    """[8, 4096, 4096] as eight 32 MiB allocations: same bits as the stacked launch."""
    W = 8
    g = torch.Generator(device="cpu").manual_seed(3)
    bufs = [torch.randn(4096, 4096, generator=g).to(BF16).to(dev) for _ in range(W)]
    stack = torch.stack(bufs)
    assert same_bits(comm.one_shot_all_reduce(bufs), comm.one_shot_all_reduce(stack))
    del stack


@pytest.mark.parametrize("rank", [0, 3, 7])
def test_two_shot_row_share(dev, rank):
    W = 8
    stack = orc.make_stack(W, (64, 256))
    share = comm.two_shot_all_reduce(stack.to(dev), rank=rank)
    assert share.shape == (8, 256)
    assert same_bits(share, orc.reduce(stack[:, rank * 8:(rank + 1) * 8]))
    full = comm.two_shot_all_reduce(stack.to(dev), rank=None)
    assert same_bits(full, orc.reduce(stack))
    # with bias, share only
    bias = orc.randn_bf16((64, 256), 3)
    out = torch.empty(8, 256, dtype=BF16, device=dev)
    fused.two_shot_all_reduce_bias(stack.to(dev), None, bias.to(dev), out, rank=rank)
    assert same_bits(out, orc.reduce(stack, bias, bias_first=False)[rank * 8:(rank + 1) * 8])
    vb = orc.randn_bf16((256,), 4)
    fused.two_shot_all_reduce_bias(stack.to(dev), None, vb.to(dev), out, rank=rank)
    assert same_bits(out, orc.reduce(stack, vb, bias_first=False)[rank * 8:(rank + 1) * 8])


@pytest.mark.parametrize("numel,block", [(8 * 37 * 16, 64), (2048 * 8 * 3, 2048), (8 * 1000, 2048)])
def test_two_shot_striped_share(dev, numel, block):
    W = 8
    stack = orc.make_stack(W, (numel,))
    bias = orc.randn_bf16((numel,), 9)
    full = orc.reduce(stack, bias, bias_first=False)
    assembled = torch.empty_like(full)
    for rank in range(W):
        idx = orc.striped_indices(numel, W, block, rank)
        share = comm.two_shot_all_reduce(stack.to(dev), rank=rank, layout="striped", BLOCK_SIZE=block)
        assert share.numel() == idx.numel()
        if idx.numel():
            assert same_bits(share, orc.reduce_striped(stack, None, block, rank))
        out = torch.empty(idx.numel(), dtype=BF16, device=dev)
        fused.two_shot_all_reduce_bias(stack.to(dev), None, bias.to(dev), out, BLOCK_SIZE=block, rank=rank,
                                       layout="striped", numel=numel)
        assembled[idx] = out.cpu()
    assert same_bits(assembled, full)


def test_rotated_band_reduce(dev):
    from kraken_amd.fused.gemm_reduce_scatter_ce_persistent import reduce as rotated_reduce
    W, rows, N = 8, 24, 264
    inp = orc.randn_bf16((W * rows, N), 33)
    for rank in (0, 5):
        for fp32_acc in (False, True):
            out = torch.empty(rows, N, dtype=BF16, device=dev)
            rotated_reduce(inp.to(dev), out, {"RANK": rank, "WORLD_SIZE": W, "fp32_acc": fp32_acc})
            assert same_bits(out, orc.reduce_rotated(inp, W, rank, acc_bf16=not fp32_acc))


def test_full_size_config2(dev):
    """benchmark config 2: stack [8,4096,4096] -> [4096,4096], and the two-shot 1/8 row chunk.
    Checked exactly against the oracle on sampled row bands, and by linearity on the whole."""
    W, R, D = 8, 4096, 4096
    g = torch.Generator(device="cpu"); g.manual_seed(42)
    stack = torch.randn((W, R, D), generator=g, dtype=torch.float32).to(BF16)
    sd = stack.to(dev)
    out = comm.one_shot_all_reduce(sd)
    for r0 in (0, 1337, 4096 - 64):
        assert same_bits(out[r0:r0 + 64], orc.reduce(stack[:, r0:r0 + 64]))
    share = comm.two_shot_all_reduce(sd, rank=5)
    assert share.shape == (512, 4096)
    assert same_bits(share, out[5 * 512:6 * 512])
    # size-independent property: the sum of all outputs equals the sum of all inputs
    tot_in = sd.float().sum(dtype=torch.float64)
    tot_out = out.float().sum(dtype=torch.float64)
    assert abs(float(tot_in - tot_out)) <= 2e-2 * float(sd.float().abs().sum(dtype=torch.float64)) * 2 ** -7
    # swapping two slices leaves the result within one rounding
    sd2 = sd.clone(); sd2[[0, 7]] = sd[[7, 0]]
    torch.testing.assert_close(comm.one_shot_all_reduce(sd2).float(), out.float(), rtol=2 ** -7, atol=1e-5)


def test_reduce_paths_replay_from_a_graph(dev):
    """The reduce and row entry points enqueue kernels only: captured once, every replay (with
    eager work in between) reproduces the eager result bit for bit."""
    W, rows, D = 8, 48, 5120
    stack = orc.make_stack(W, (rows, D)).to(dev)
    bias, w = orc.make_bias_weight(D)
    bias, w = bias.to(dev), w.to(dev)
    out = torch.empty(rows, D, dtype=BF16, device=dev)
    y = torch.empty(rows, D, dtype=BF16, device=dev)

    def run():
        s1 = comm.one_shot_all_reduce(stack)
        s2 = comm.two_shot_all_reduce(stack, rank=2)
        fused.one_shot_all_reduce_bias(stack, None, bias.expand(rows, D).contiguous(), out)
        fused.one_shot_all_reduce_bias_rms_norm(stack, None, bias, w, y)
        return s1, s2, out, y

    eager = [t.clone() for t in run()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            got = run()
    for rep in range(3):
        for t in got:
            t.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for e, r in zip(eager, got):
            assert torch.equal(e, r)


def test_benchmark_helpers(dev):
    """The reference's two timing methods (kraken/_logging/benchmarking.py): per-call events and
    profiler events matched by kernel name; both with the reference's keywords."""
    from kraken_amd._logging import benchmark_with_event, benchmark_with_profiler
    stack = orc.make_stack(8, (256, 4096)).to(dev)
    fn = lambda: comm.one_shot_all_reduce(stack)                      # noqa: E731
    t_event = benchmark_with_event(fn, warmup_iters=5, benchmark_iters=10, flush_l2=True)
    t_graph = benchmark_with_event(fn, warmup_iters=5, benchmark_iters=10, flush_l2=False, cuda_graph=True)
    t_index = benchmark_with_event(lambda i: comm.one_shot_all_reduce(stack), warmup_iters=2, benchmark_iters=5)
    assert 0.5 < t_event < 500 and 0.5 < t_graph < 500 and 0.5 < t_index < 500
    t_prof = benchmark_with_profiler(fn, r".*reduce_kernel.*", warmup_iters=5, benchmark_iters=10)
    assert 0.5 < t_prof < 500
    assert benchmark_with_profiler(fn, r"no such kernel", warmup_iters=1, benchmark_iters=2) == 0.0



def _device_kernels(fn):
    """Names of the device kernels (and device copies) one call of fn enqueues."""
    from torch.profiler import ProfilerActivity, profile

    fn()
    torch.cuda.synchronize()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        fn()
        torch.cuda.synchronize()
    return [e.name for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA]


def test_input_is_read_in_place_by_one_kernel(dev):
    """The reference stages this rank's input into its symmetric buffer inside the kernel
    (kraken/fused/one_shot_all_reduce_bias.py:56-65).  Here the input is the rank's source where
    it lies: one launch, no copy, the staged form's bits; stage=True keeps the side effect."""
    W, rows, D, rank = 8, 16, 5120, 3
    stack = orc.make_stack(W, (rows, D), seed0=5)
    x = orc.randn_bf16((rows, D), 77)
    bias, w = orc.randn_bf16((rows, D), 9), orc.randn_bf16((D,), 4, 0.02, 1.0)
    staged = stack.clone()
    staged[rank] = x
    buf = torch.zeros(W, 1024, 1024, dtype=BF16, device=dev)          # larger than the message, as in the reference's tests
    for r in range(W):
        buf[r].view(-1)[: rows * D].copy_(stack[r].view(-1))
    before = buf.clone()
    xd, bd, wd = x.to(dev), bias.to(dev), w.to(dev)
    out = torch.empty(rows, D, dtype=BF16, device=dev)
    y = torch.empty(rows, D, dtype=BF16, device=dev)
    calls = {
        "one_shot_bias": lambda **kw: fused.one_shot_all_reduce_bias(buf, xd, bd, out, rank=rank, **kw),
        "two_shot_bias": lambda **kw: fused.two_shot_all_reduce_bias(buf, xd, bd, out, rank=rank, **kw),
        "one_shot_rms": lambda **kw: fused.one_shot_all_reduce_bias_rms_norm(buf, xd, bd, wd, y, rank=rank, **kw),
        "two_shot_rms": lambda **kw: fused.two_shot_all_reduce_bias_rms_norm(buf, xd, bd, wd, y, rank=rank, **kw),
    }
    wants = {
        "one_shot_bias": orc.reduce(staged, bias, bias_first=True),
        "two_shot_bias": orc.reduce(staged, bias, bias_first=False),
    }
    for name, call in calls.items():
        res = y if name.endswith("rms") else out
        res.zero_()
        kernels = _device_kernels(call)
        assert len(kernels) == 1, kernels                              # no copy kernel, no memcpy
        assert torch.equal(buf, before)                                # the buffer is left alone
        in_place = res.clone()
        if name in wants:
            assert same_bits(in_place, wants[name])
        else:
            torch.testing.assert_close(in_place.cpu(), orc.reduce_bias_rms_norm(staged, bias, w), rtol=2e-2, atol=2e-2)
        res.zero_()
        kernels = _device_kernels(lambda: call(stage=True))
        assert len(kernels) == 2, kernels                              # the copy-in, then the kernel
        assert torch.equal(res, in_place)                              # the same bits
        assert torch.equal(buf[rank].view(-1)[: rows * D], xd.view(-1))
        buf.copy_(before)
