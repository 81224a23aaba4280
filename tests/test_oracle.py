"""Pins of the CPU oracle (oracle/oracle.py): independent C restatement, library routines,
closed forms and brute force.  No GPU, no reference import."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as orc

BF16 = torch.bfloat16


def u16(t):
    return t.contiguous().view(torch.int16)


# ------------------------------------------------------------------ W-way reduce
@pytest.mark.parametrize("W", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("bias_mode", ["none", "full", "vector"])
@pytest.mark.parametrize("bias_first", [True, False])
def test_reduce_matches_c_restatement_bit_for_bit(oracle_c, W, bias_mode, bias_first):
    rows, D = 5, 64
    stack = orc.make_stack(W, (rows, D), seed0=7)
    bias = None
    if bias_mode == "full":
        bias = orc.randn_bf16((rows, D), 99)
    elif bias_mode == "vector":
        bias = orc.randn_bf16((D,), 99)
    got = orc.reduce(stack, bias, bias_first)
    out = torch.empty(rows * D, dtype=torch.int16)
    oracle_c.orc_reduce(
        u16(stack).data_ptr(), W, rows * D, rows * D,
        None if bias is None else u16(bias).data_ptr(), 0 if bias is None else bias.numel(),
        int(bias_first), out.data_ptr(),
    )
    assert torch.equal(u16(got).reshape(-1), out)


def test_reduce_closed_form_rank_multiples():
    # slices = (r+1)*c  =>  c * W(W+1)/2   (adapts test/test_gemm_allreduce.py:92-117)
    W, c = 8, 0.5
    stack = torch.stack([torch.full((4, 16), (r + 1) * c, dtype=BF16) for r in range(W)])
    assert torch.equal(orc.reduce(stack).float(), torch.full((4, 16), c * W * (W + 1) / 2))


def test_reduce_w1_is_identity_and_bias_none_is_plain_sum():
    x = orc.make_stack(1, (3, 32))
    assert torch.equal(orc.reduce(x), x[0])
    s = orc.make_stack(4, (3, 32))
    assert torch.equal(orc.reduce(s, None, True), orc.reduce(s, None, False))


def test_reduce_vector_bias_equals_expanded_full_bias():
    s = orc.make_stack(8, (6, 32))
    b = orc.randn_bf16((32,), 5)
    assert torch.equal(orc.reduce(s, b), orc.reduce(s, b.expand(6, 32).contiguous()))


def test_reduce_brute_force_tiny():
    W = 4
    s = orc.make_stack(W, (8,))
    b = orc.randn_bf16((8,), 1)
    want = []
    for i in range(8):
        acc = torch.tensor(float(b[i]), dtype=torch.float32)
        for r in range(W):
            acc = acc + torch.tensor(float(s[r, i]), dtype=torch.float32)
        want.append(acc.to(BF16))
    assert torch.equal(orc.reduce(s, b), torch.stack(want))


def test_reduce_library_form_within_fp32_reassociation():
    s = orc.make_stack(8, (64, 128))
    b = orc.randn_bf16((128,), 3, 0.02)
    a, l = orc.reduce(s, b).float(), orc.reduce_library(s, b).float()
    # at most one bf16 ulp apart (a different fp32 order can flip one rounding)
    assert ((a - l).abs() <= a.abs() * 2.0 ** -7 + 1e-30).all()
    assert (a == l).float().mean() > 0.99


def test_reduce_permutation_of_slices_is_immaterial_at_tolerance():
    s = orc.make_stack(8, (16, 64))
    p = s[torch.tensor([3, 1, 7, 0, 2, 6, 5, 4])]
    torch.testing.assert_close(orc.reduce(s).float(), orc.reduce(p).float(), rtol=2 ** -7, atol=1e-6)


def test_striped_ownership_partitions_the_input():
    numel, W, block = 8 * 37, 4, 16      # ragged last stripe
    seen = torch.zeros(numel, dtype=torch.int32)
    for r in range(W):
        idx = orc.striped_indices(numel, W, block, r)
        seen[idx] += 1
        # owned offsets are  stripe*block*W + r*block + [0, block)
        assert ((idx % (block * W)) // block == r).all()
    assert (seen == 1).all()


def test_striped_shares_assemble_to_full_reduce():
    W, block = 4, 16
    s = orc.make_stack(W, (8 * 37,))
    b = orc.randn_bf16((8 * 37,), 11)
    full = orc.reduce(s, b, bias_first=False)
    out = torch.empty_like(full)
    for r in range(W):
        out[orc.striped_indices(full.numel(), W, block, r)] = orc.reduce_striped(s, b, block, r)
    assert torch.equal(out, full)


def test_reduce_rotated_order_and_rounding():
    W, rows, N = 4, 3, 16
    inp = orc.randn_bf16((W * rows, N), 21)
    # fp32 accumulation: order is immaterial at tolerance, equals plain band sum
    plain = inp.reshape(W, rows, N).float().sum(0)
    torch.testing.assert_close(orc.reduce_rotated(inp, W, 1, acc_bf16=False).float(), plain, rtol=2 ** -7, atol=1e-6)
    # bf16 accumulation, spelled out for rank 2: bands 3, 0, 1, 2
    b = inp.reshape(W, rows, N)
    acc = b[3]
    for j in (0, 1, 2):
        acc = (acc.float() + b[j].float()).to(BF16)
    assert torch.equal(orc.reduce_rotated(inp, W, 2, acc_bf16=True), acc)


# ------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("D", [64, 4096, 5120])
def test_rms_norm_bit_identical_to_library_routine(D):
    x = orc.randn_bf16((7, D), 4)
    w = orc.randn_bf16((D,), 5)
    assert torch.equal(orc.rms_norm(x, w, 1e-5), F.rms_norm(x, (D,), w, 1e-5))


def test_rms_norm_closed_forms():
    D, eps = 256, 1e-5
    w = orc.randn_bf16((D,), 6, 0.02, 1.0)
    c = 3.0
    x = torch.full((2, D), c, dtype=BF16)
    want = (w.float() * (c / math.sqrt(c * c + eps))).to(BF16)
    assert torch.equal(orc.rms_norm(x, w, eps)[0], want)
    assert torch.equal(orc.rms_norm(torch.zeros(2, D, dtype=BF16), w, eps), torch.zeros(2, D, dtype=BF16))
    ones = torch.ones(D, dtype=BF16)
    y = orc.rms_norm(orc.randn_bf16((4, D), 8), ones, eps).float()
    torch.testing.assert_close((y * y).mean(-1), torch.ones(4), rtol=1e-2, atol=1e-2)
    xs = orc.randn_bf16((4, D), 9)
    torch.testing.assert_close(orc.rms_norm(xs, w, eps).float(), orc.rms_norm(xs * 4, w, eps).float(),
                               rtol=2 ** -7, atol=1e-6)  # scale invariance (power of two: exact inputs)


@pytest.mark.parametrize("bias_mode", ["none", "full", "vector"])
def test_reduce_bias_rms_norm_against_c_and_library(oracle_c, bias_mode):
    W, rows, D, eps = 8, 6, 320, 1e-5
    stack = orc.make_stack(W, (rows, D), seed0=50)
    w = orc.randn_bf16((D,), 51, 0.02, 1.0)
    bias = {"none": None, "full": orc.randn_bf16((rows, D), 52), "vector": orc.randn_bf16((D,), 52, 0.02)}[bias_mode]
    got = orc.reduce_bias_rms_norm(stack, bias, w, eps)
    lib = orc.reduce_bias_rms_norm_library(stack, bias, w, eps)
    y = torch.empty(rows * D, dtype=torch.int16)
    scratch = torch.empty(D, dtype=torch.float32)
    oracle_c.orc_reduce_rmsnorm(
        u16(stack).data_ptr(), W, rows * D, rows, D, None if bias is None else u16(bias).data_ptr(),
        int(bias_mode == "vector"), u16(w).data_ptr(), eps, y.data_ptr(), scratch.data_ptr(),
    )
    cy = y.view(BF16).reshape(rows, D)
    # The C version sums the squares in double and uses 1/sqrt; the torch forms differ from it
    # and from each other by fp32 rounding of rstd only: at most one bf16 ulp, rarely.
    for other in (cy, lib):
        d = (got.float() - other.float()).abs()
        assert (d <= got.float().abs() * 2.0 ** -7 + 1e-30).all()
        assert (d == 0).float().mean() > 0.98


def test_reduce_bias_rms_norm_composes():
    W, rows, D = 4, 5, 128
    stack = orc.make_stack(W, (rows, D))
    b, w = orc.make_bias_weight(D)
    # W = 1, no bias: the fused form is the stand-alone norm
    assert torch.equal(orc.reduce_bias_rms_norm(stack[:1], None, w), orc.rms_norm(stack[0], w))
    # norm of the fp32 reduced row, redone by hand
    s = b.float() + stack[0].float()
    for r in range(1, W):
        s = s + stack[r].float()
    want = (s * torch.rsqrt((s * s).mean(-1, keepdim=True) + 1e-5) * w.float())
    torch.testing.assert_close(orc.reduce_bias_rms_norm(stack, b, w).float(), want, rtol=2 ** -7, atol=1e-6)


# ------------------------------------------------------------------ GEMM + reduce
def test_gemm_rank_specific_known_answer():
    # test/test_gemm_allreduce.py:92-117: a = (rank+1)*ones, b = ones  =>  K * sum(1..W), exactly
    M = N = K = 32
    W = 4
    b = torch.ones(K, N, dtype=BF16)
    a0 = torch.ones(M, K, dtype=BF16)
    peers = torch.stack([torch.full((M, N), float((r + 1) * K), dtype=BF16) for r in range(1, W)])
    out = orc.gemm_all_reduce(a0, b, peers)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out, torch.full((M, N), float(K * 10)), rtol=1e-5, atol=1e-5)


def test_gemm_reduce_scatter_rank_specific_known_answer():
    # test/test_gemm_reduce_scatter.py:76-91 with W = 4, rank r: every element K * 10
    M, N, K, W = 64, 32, 16, 4
    for rank in range(W):
        a = torch.full((M, K), float(rank + 1), dtype=BF16)
        b = torch.ones(K, N, dtype=BF16)
        others = [r for r in range(W) if r != rank]
        peers = torch.stack([torch.full((M // W, N), float((r + 1) * K), dtype=BF16) for r in others])
        out, c = orc.gemm_reduce_scatter(a, b, peers, rank, W)
        assert out.shape == (M // W, N)
        assert torch.equal(out.float(), torch.full((M // W, N), float(K * 10)))
        assert torch.equal(c.float(), torch.full((M, N), float((rank + 1) * K)))


def test_gemm_identity_and_ones():
    a = orc.randn_bf16((24, 16), 1)
    assert torch.equal(orc.gemm_all_reduce(a, torch.eye(16, dtype=BF16)), a.float())
    assert torch.equal(orc.gemm_all_reduce(torch.ones(8, 40, dtype=BF16), torch.ones(40, 8, dtype=BF16)),
                       torch.full((8, 8), 40.0))


def test_gemm_against_c_triple_loop(oracle_c):
    M, N, K, P = 16, 8, 16, 3
    a, b = orc.randn_bf16((M, K), 1), orc.randn_bf16((K, N), 2, 0.02)
    peers = torch.stack([orc.randn_bf16((M, N), 100 + j) for j in range(P)])
    bias = orc.randn_bf16((N,), 42, 0.02)
    got = orc.gemm_all_reduce(a, b, peers, bias)
    c = torch.empty(M, N, dtype=torch.float32)
    oracle_c.orc_gemm(u16(a).data_ptr(), u16(b).data_ptr(), M, N, K, u16(peers).data_ptr(), P,
                      u16(bias).data_ptr(), c.data_ptr())
    torch.testing.assert_close(got, c, rtol=1e-5, atol=1e-5)


def test_reduce_scatter_band_is_slice_of_all_reduce():
    M, N, K, W = 64, 24, 32, 4
    a, b = orc.randn_bf16((M, K), 1), orc.randn_bf16((K, N), 2)
    full_peers = torch.stack([orc.randn_bf16((M, N), 100 + j) for j in range(W - 1)])
    full = orc.gemm_all_reduce(a, b, full_peers)
    for rank in range(W):
        rows = slice(rank * M // W, (rank + 1) * M // W)
        out, _ = orc.gemm_reduce_scatter(a, b, full_peers[:, rows].contiguous(), rank, W, torch.float32)
        torch.testing.assert_close(out, full[rows], rtol=1e-6, atol=1e-6)


def test_all_gather_matmul_exact_gather():
    stack = orc.make_stack(4, (8, 16))
    b = orc.randn_bf16((16, 8), 3)
    a_full, c = orc.all_gather_matmul(stack, b)
    assert torch.equal(a_full, torch.cat(list(stack), 0))
    torch.testing.assert_close(c.float(), torch.cat([s.float() @ b.float() for s in stack], 0), rtol=2 ** -7, atol=1e-5)


def test_all_gather_matmul_fp8_pins():
    """fp8 operands, fp32 accumulate, one rounding to fp8: closed forms, saturation at 448, and for
    random operands the nearest representable value found by searching the table of all finite
    e4m3 codes (ties to the even code) around the product computed exactly in float64."""
    fp8 = torch.float8_e4m3fn
    W, m, K, N = 4, 8, 32, 16
    # closed forms on exactly representable values: every element K * s * t
    for s_, t_, want in ((0.5, 0.25, 4.0), (1.5, 2.0, 96.0), (2.0, 8.0, 448.0), (16.0, 16.0, 448.0), (-16.0, 16.0, -448.0)):
        a = torch.full((W, m, K), s_).to(fp8)
        b = torch.full((K, N), t_).to(fp8)
        a_full, c = orc.all_gather_matmul_fp8(a, b)
        assert c.dtype == fp8 and torch.equal(a_full.view(torch.uint8), a.reshape(W * m, K).view(torch.uint8))
        assert torch.equal(c.float(), torch.full((W * m, N), want)), (s_, t_)
    # the table of finite codes, by its definition: (-1)^s 2^(e-7) (1 + f/8), subnormals f/8 * 2^-6
    vals = []
    for code in range(256):
        e, f = (code >> 3) & 15, code & 7
        if e == 15 and f == 7:
            continue
        v = (f / 8.0) * 2.0 ** -6 if e == 0 else (1 + f / 8.0) * 2.0 ** (e - 7)
        vals.append((-v if code & 0x80 else v, code))
    table = torch.tensor([v for v, _ in vals], dtype=torch.float64)
    codes = torch.tensor([c for _, c in vals])
    assert torch.equal(codes.to(torch.uint8).view(fp8).double(), table)          # torch's decoding agrees with the definition
    g = torch.Generator().manual_seed(5)
    scale = torch.tensor([32.0, 2.0, 0.25, 1.0 / 64]).reshape(W, 1, 1)            # saturating, ordinary and tiny rows
    a = (torch.randn(W, m, K, generator=g) * scale).to(fp8)
    b = (torch.randn(K, N, generator=g) * 3).to(fp8)
    _, c = orc.all_gather_matmul_fp8(a, b)
    exact = a.reshape(W * m, K).double() @ b.double()                             # exact: 8-bit significands, 32 terms
    dist = (exact.reshape(-1, 1) - table.reshape(1, -1)).abs()
    best = dist.min(dim=1).values
    near = dist <= best.reshape(-1, 1)                                            # one candidate, or two at a tie
    got = c.reshape(-1).view(torch.uint8).to(torch.int64)
    for i in range(got.numel()):
        cand = codes[near[i]]
        if exact.reshape(-1)[i].abs() >= 448:
            assert (int(got[i]) & 0x7f) == 0x7e
        elif cand.numel() == 1:
            assert int(got[i]) == int(cand[0]) or (float(exact.reshape(-1)[i]) == 0.0 and (int(got[i]) & 0x7f) == 0)
        else:
            assert int(got[i]) in [int(x) for x in cand if int(x) % 2 == 0]
    assert (exact.abs() >= 448).any() and (exact.abs() < 1).any()                # both ends of the range are exercised


def test_known_answers_of_the_reference_tests():
    """tests/golden/known_answers.json: the closed-form cases of the reference's tests, against the oracle."""
    import json
    import pathlib

    cases = {c["name"]: c for c in json.loads((pathlib.Path(__file__).parent / "golden" / "known_answers.json").read_text())["cases"]}
    c = cases["gemm_all_reduce_rank_specific"]
    W, M, N, K = c["world_size"], c["M"], c["N"], c["K"]
    b = torch.ones(K, N, dtype=torch.bfloat16)
    partials = [(torch.full((M, K), float(r + 1), dtype=torch.bfloat16).float() @ b.float()).to(torch.bfloat16) for r in range(W)]
    out = orc.gemm_all_reduce(torch.full((M, K), 1.0, dtype=torch.bfloat16), b, torch.stack(partials[1:]))
    torch.testing.assert_close(out, torch.full((M, N), c["expected_value"]), rtol=c["tolerance"], atol=c["tolerance"])
    c = cases["gemm_reduce_scatter_rank_specific"]
    W, M, N, K = c["world_size"], c["M"], c["N"], c["K"]
    b = torch.ones(K, N, dtype=torch.bfloat16)
    for rank in range(W):
        a = torch.full((M, K), float(rank + 1), dtype=torch.bfloat16)
        peers = torch.stack([torch.full((M // W, N), float((r + 1) * K), dtype=torch.bfloat16) for r in range(W) if r != rank])
        out, _ = orc.gemm_reduce_scatter(a, b, peers, rank, W)
        assert torch.equal(out.float(), torch.full((M // W, N), c["expected_value"]))

