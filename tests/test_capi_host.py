"""Host side of the C ABI, exercised without a GPU: the library loads, exports every symbol
include/kraken_amd.h declares, and rejects bad arguments before any launch.  The Python
wrappers raise like the reference's asserts and refuse host tensors (no CPU fallback)."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

import kraken_amd
from kraken_amd import _lib, comm, fused

ROOT = Path(__file__).resolve().parent.parent
BF16 = torch.bfloat16
FAKE = 0x10000  # aligned, non-null; never dereferenced because validation fails first


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def test_library_exports_every_declared_symbol(lib):
    header = (ROOT / "include" / "kraken_amd.h").read_text()
    declared = set(re.findall(r"\b(kr_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(_lib.EXPORTS)
    raw = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared:
        assert hasattr(raw, name), f"{name} not exported"
    assert lib.kr_version() >= 100


def test_strerror_known_and_unknown(lib):
    assert "128-bit" in _lib.strerror(_lib.KR_ERR_NUMEL_MOD8)
    assert _lib.strerror(0) == "success"
    assert "unknown" in _lib.strerror(-999)


def test_reduce_argument_errors(lib):
    f = lib.kr_reduce_bf16
    assert f(FAKE, 8, 64, 12, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_NUMEL_MOD8
    assert f(FAKE, 0, 64, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_WORLD_SIZE
    assert f(FAKE, 17, 64, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_WORLD_SIZE
    assert f(None, 8, 64, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_NULL_POINTER
    assert f(FAKE, 8, 64, 16, None, 0, 0, 1, None, None) == _lib.KR_ERR_NULL_POINTER
    assert f(FAKE + 2, 8, 64, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_ALIGNMENT
    assert f(FAKE, 8, 60, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_ALIGNMENT
    assert f(FAKE, 8, 64, -8, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_BAD_DIM
    assert f(FAKE, 8, 64, 64, FAKE, 24, 16, 1, FAKE, None) == _lib.KR_ERR_BIAS_SHAPE
    assert f(FAKE, 8, 64, 64, FAKE + 4, 64, 16, 1, FAKE, None) == _lib.KR_ERR_ALIGNMENT
    # empty input: nothing to do, nothing launched
    assert f(None, 8, 0, 0, None, 0, 0, 1, None, None) == 0


def test_rmsnorm_argument_errors(lib):
    f = lib.kr_reduce_rmsnorm_bf16
    assert f(FAKE, 8, 4096, 1, 4100, None, 0, FAKE, 1e-5, FAKE, None) == _lib.KR_ERR_NUMEL_MOD8
    assert f(FAKE, 8, 1 << 20, 1, 65536 + 8, None, 0, FAKE, 1e-5, FAKE, None) == _lib.KR_ERR_ROW_TOO_LONG
    assert f(FAKE, 8, 4096, 1, 4096, None, 0, None, 1e-5, FAKE, None) == _lib.KR_ERR_NULL_POINTER
    assert f(FAKE, 99, 4096, 1, 4096, None, 0, FAKE, 1e-5, FAKE, None) == _lib.KR_ERR_WORLD_SIZE
    assert f(FAKE, 8, 4096, 0, 4096, None, 0, FAKE, 1e-5, FAKE, None) == 0
    g = lib.kr_rmsnorm_bf16
    assert g(FAKE, FAKE, 1e-5, 4, 0, FAKE, None) == _lib.KR_ERR_BAD_DIM
    assert g(FAKE, FAKE + 8, 1e-5, 4, 64, FAKE, None) == _lib.KR_ERR_ALIGNMENT


def test_rmsnorm_workspace_entries(lib, monkeypatch):
    """Which shapes the split-row kernel takes (a few long rows), and that the workspace forms
    validate like the plain ones."""
    q = lib.kr_rmsnorm_workspace_bytes
    need = q(8, 16, 8192)
    assert need > 0 and q(8, 1, 8192) == need and q(4, 16, 32768) == need
    assert q(8, 256, 4096) == 0 and q(8, 16, 1024) == 0 and q(3, 16, 8192) == 0 and q(8, 128, 8192) == 0
    assert q(8, 16, 8190) == 0 and q(8, 0, 8192) == 0 and q(8, 2, 65536) == 0
    f = lib.kr_reduce_rmsnorm_ws_bf16
    assert f(FAKE, 8, 8192 * 16, 16, 8192, None, 0, FAKE, 1e-5, FAKE, FAKE + 8, need, None, None) == _lib.KR_ERR_ALIGNMENT
    assert f(FAKE, 8, 8192 * 16, 16, 8196, None, 0, FAKE, 1e-5, FAKE, FAKE, need, None, None) == _lib.KR_ERR_NUMEL_MOD8
    assert f(None, 8, 8192 * 16, 16, 8192, None, 0, FAKE, 1e-5, FAKE, FAKE, need, None, None) == _lib.KR_ERR_NULL_POINTER
    # the status word of the bounded exchange: 4-byte aligned or NULL
    assert f(FAKE, 8, 8192 * 16, 16, 8192, None, 0, FAKE, 1e-5, FAKE, FAKE, need, FAKE + 2, None) == _lib.KR_ERR_ALIGNMENT
    assert f(FAKE, 8, 8192 * 16, 0, 8192, None, 0, FAKE, 1e-5, FAKE, FAKE, need, FAKE, None) == 0
    g = lib.kr_reduce_rmsnorm_ptrs_ws_bf16
    assert g(None, 8, 16, 8192, None, 0, FAKE, 1e-5, FAKE, FAKE, need, None, None) == _lib.KR_ERR_NULL_POINTER
    monkeypatch.setenv("KRAKEN_AMD_ROW_SPLIT", "0")
    assert q(8, 16, 8192) == 0
    monkeypatch.setenv("KRAKEN_AMD_ROW_SPLIT", "1")
    assert q(8, 64, 1024) == need and q(8, 65, 1024) == 0 and q(8, 1, 512) == 0   # 64 rows at most, two wavefronts at least


def test_gemm_argument_errors(lib):
    f = lib.kr_gemm_reduce_bf16

    def call(**kw):
        a = dict(A=FAKE, lda_m=64, lda_k=1, B=FAKE, ldb_k=64, ldb_n=1, M=64, N=64, K=64, peers=None,
                 n_peers=0, pstride=0, bias=None, band0=0, band=64, c_full=None, out=FAKE, f32=0, pivot=0)
        a.update(kw)
        return f(a["A"], a["lda_m"], a["lda_k"], a["B"], a["ldb_k"], a["ldb_n"], a["M"], a["N"], a["K"],
                 a["peers"], a["n_peers"], a["pstride"], a["bias"], a["band0"], a["band"], a["c_full"],
                 a["out"], a["f32"], a["pivot"], None)

    assert call(K=60) == _lib.KR_ERR_NUMEL_MOD8
    assert call(N=60) == _lib.KR_ERR_NUMEL_MOD8
    assert call(lda_k=2) == _lib.KR_ERR_LAYOUT
    assert call(ldb_k=3, ldb_n=5) == _lib.KR_ERR_LAYOUT
    assert call(band0=32, band=64) == _lib.KR_ERR_BAND
    assert call(A=None) == _lib.KR_ERR_NULL_POINTER
    assert call(out=None) == _lib.KR_ERR_NULL_POINTER
    assert call(n_peers=3, peers=None) == _lib.KR_ERR_NULL_POINTER
    assert call(n_peers=3, peers=FAKE, pstride=64) == _lib.KR_ERR_BAD_DIM
    assert call(lda_m=68) == _lib.KR_ERR_ALIGNMENT
    assert call(M=-1) == _lib.KR_ERR_BAD_DIM
    assert call(M=0, band=0) == 0


def _table(*ptrs):
    return (ctypes.c_void_p * len(ptrs))(*ptrs)


def test_pointer_table_argument_errors(lib):
    """The kr_*_ptrs_bf16 forms reject what their stacked forms reject, and a bad table entry."""
    good = _table(*[FAKE + 4096 * r for r in range(8)])
    f = lib.kr_reduce_ptrs_bf16
    assert f(good, 8, 12, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_NUMEL_MOD8
    assert f(good, 0, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_WORLD_SIZE
    assert f(good, 17, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_WORLD_SIZE
    assert f(None, 8, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_NULL_POINTER
    assert f(good, 8, 16, None, 0, 0, 1, None, None) == _lib.KR_ERR_NULL_POINTER
    assert f(_table(FAKE, None), 2, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_NULL_POINTER
    assert f(_table(FAKE, FAKE + 8), 2, 16, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_ALIGNMENT
    assert f(good, 8, 64, FAKE, 24, 16, 1, FAKE, None) == _lib.KR_ERR_BIAS_SHAPE
    assert f(good, 8, -8, None, 0, 0, 1, FAKE, None) == _lib.KR_ERR_BAD_DIM
    assert f(None, 8, 0, None, 0, 0, 1, None, None) == 0

    f = lib.kr_reduce_striped_ptrs_bf16
    assert f(good, 8, 4096, None, 12, 0, FAKE, None) == _lib.KR_ERR_STRIPE
    assert f(good, 8, 4096, None, 256, 8, FAKE, None) == _lib.KR_ERR_STRIPE
    assert f(_table(FAKE, FAKE + 2), 2, 4096, None, 256, 0, FAKE, None) == _lib.KR_ERR_ALIGNMENT
    assert f(None, 8, 4096, None, 256, 0, FAKE, None) == _lib.KR_ERR_NULL_POINTER
    assert f(good, 8, 256, None, 256, 3, FAKE, None) == 0   # rank 3 owns nothing of a 256-element input

    f = lib.kr_reduce_rmsnorm_ptrs_bf16
    assert f(good, 8, 1, 4100, None, 0, FAKE, 1e-5, FAKE, None) == _lib.KR_ERR_NUMEL_MOD8
    assert f(good, 8, 1, 65536 + 8, None, 0, FAKE, 1e-5, FAKE, None) == _lib.KR_ERR_ROW_TOO_LONG
    assert f(good, 8, 1, 4096, None, 0, None, 1e-5, FAKE, None) == _lib.KR_ERR_NULL_POINTER
    assert f(None, 8, 1, 4096, None, 0, FAKE, 1e-5, FAKE, None) == _lib.KR_ERR_NULL_POINTER
    assert f(_table(FAKE + 6), 1, 1, 4096, None, 0, FAKE, 1e-5, FAKE, None) == _lib.KR_ERR_ALIGNMENT
    assert f(good, 8, 0, 4096, None, 0, None, 1e-5, None, None) == 0

    f = lib.kr_gemm_reduce_ptrs_bf16
    def args(**kw):
        a = dict(A=FAKE, lda_m=64, lda_k=1, B=FAKE, ldb_k=64, ldb_n=1, M=64, N=64, K=64, peers=None, n_peers=0,
                 bias=None, band_row0=0, band_rows=64, c_full=None, out=FAKE, out_is_fp32=0, tile_pivot=0,
                 stream=None)
        a.update(kw)
        return tuple(a.values())
    assert f(*args(n_peers=2, peers=None)) == _lib.KR_ERR_NULL_POINTER
    assert f(*args(n_peers=2, peers=_table(FAKE, None))) == _lib.KR_ERR_NULL_POINTER
    assert f(*args(n_peers=2, peers=_table(FAKE, FAKE + 4))) == _lib.KR_ERR_ALIGNMENT
    assert f(*args(n_peers=16, peers=good)) == _lib.KR_ERR_WORLD_SIZE
    assert f(*args(n_peers=2, peers=good, band_row0=32, band_rows=64)) == _lib.KR_ERR_BAND
    assert f(*args(n_peers=2, peers=good, lda_k=2)) == _lib.KR_ERR_LAYOUT
    assert f(*args(n_peers=2, peers=good, M=0, band_rows=0)) == 0


def test_wrappers_accept_a_list_of_buffers_and_check_it():
    bufs = [torch.zeros(4, 16, dtype=BF16) for _ in range(3)]
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        comm.one_shot_all_reduce(bufs)
    with pytest.raises(AssertionError, match="one shape"):
        comm.one_shot_all_reduce([bufs[0], torch.zeros(4, 8, dtype=BF16)])
    with pytest.raises(AssertionError, match="bfloat16"):
        comm.one_shot_all_reduce([bufs[0], torch.zeros(4, 16)])
    with pytest.raises(AssertionError, match="contiguous"):
        comm.one_shot_all_reduce([bufs[0], torch.zeros(16, 4, dtype=BF16).T])
    a = torch.zeros(8, 16, dtype=BF16)
    b = torch.zeros(16, 8, dtype=BF16)
    with pytest.raises(AssertionError, match="every peer"):
        fused.gemm_one_shot_all_reduce_fused(a, b, peers=[torch.zeros(8, 16, dtype=BF16)])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fused.gemm_one_shot_all_reduce_fused(a, b, peers=[torch.zeros(8, 8, dtype=BF16)])


def test_all_gather_matmul_argument_errors(lib):
    f = lib.kr_all_gather_matmul_bf16
    def args(**kw):
        a = dict(A=FAKE, lda_m=64, A_local=FAKE, lda_local=64, B=FAKE, ldb_k=1, ldb_n=64, M=512, N=64, K=64,
                 W=4, rank=1, splits=2, progress=FAKE, wait_us=0, status=FAKE, C=FAKE, stream=None)
        a.update(kw)
        return tuple(a.values())
    assert f(*args(W=0)) == _lib.KR_ERR_WORLD_SIZE
    assert f(*args(W=17)) == _lib.KR_ERR_WORLD_SIZE
    assert f(*args(rank=4)) == _lib.KR_ERR_STRIPE
    assert f(*args(splits=0)) == _lib.KR_ERR_STRIPE
    assert f(*args(M=500)) == _lib.KR_ERR_BAND             # 500 rows do not split into 4*2 chunks
    assert f(*args(A_local=FAKE + 2)) == _lib.KR_ERR_ALIGNMENT
    assert f(*args(lda_local=32)) == _lib.KR_ERR_LAYOUT      # shorter than K
    assert f(*args(progress=FAKE + 2)) == _lib.KR_ERR_ALIGNMENT
    assert f(*args(status=FAKE + 1)) == _lib.KR_ERR_ALIGNMENT
    assert f(*args(A=None)) == _lib.KR_ERR_NULL_POINTER
    assert f(*args(C=None)) == _lib.KR_ERR_NULL_POINTER
    assert f(*args(K=60)) == _lib.KR_ERR_NUMEL_MOD8
    assert f(*args(ldb_k=2, ldb_n=3)) == _lib.KR_ERR_LAYOUT
    assert f(*args(M=0)) == 0
    g = lib.kr_stream_write_value32
    assert g(None, 1, None) == _lib.KR_ERR_NULL_POINTER
    assert g(FAKE + 2, 1, None) == _lib.KR_ERR_ALIGNMENT


def test_gemm_row_stride_beyond_the_kernels_reach(lib):
    # a row stride of 2^24 elements: 128 rows of a tile span 4 GiB, more than the operand descriptors cover
    f = lib.kr_gemm_reduce_bf16
    assert f(FAKE, 1 << 24, 1, FAKE, 64, 1, 128, 64, 64, None, 0, 0, None, 0, 128, None, FAKE, 0, 0,
             None) == _lib.KR_ERR_LAYOUT
    assert f(FAKE, 64, 1, FAKE, 1, 1 << 24, 128, 64, 64, None, 0, 0, None, 0, 128, None, FAKE, 0, 0,
             None) == _lib.KR_ERR_LAYOUT


def test_gemm_producer_argument_errors(lib):
    f = lib.kr_gemm_producer_bf16
    def args(**kw):
        a = dict(A=FAKE, lda_m=64, lda_k=1, B=FAKE, ldb_k=64, ldb_n=1, M=512, N=64, K=64, C=FAKE, W=4, rank=1,
                 progress=FAKE, signal=FAKE, stream=None)
        a.update(kw)
        return tuple(a.values())
    assert f(*args(W=0)) == _lib.KR_ERR_WORLD_SIZE
    assert f(*args(W=17)) == _lib.KR_ERR_WORLD_SIZE
    assert f(*args(rank=4)) == _lib.KR_ERR_BAND
    assert f(*args(rank=-1)) == _lib.KR_ERR_BAND
    assert f(*args(M=510)) == _lib.KR_ERR_BAD_DIM             # 510 rows do not split into 4 bands
    assert f(*args(progress=None)) == _lib.KR_ERR_NULL_POINTER
    assert f(*args(signal=None)) == _lib.KR_ERR_NULL_POINTER
    assert f(*args(C=None)) == _lib.KR_ERR_NULL_POINTER
    assert f(*args(progress=FAKE + 2)) == _lib.KR_ERR_ALIGNMENT
    assert f(*args(signal=FAKE + 1)) == _lib.KR_ERR_ALIGNMENT
    assert f(*args(A=None)) == _lib.KR_ERR_NULL_POINTER
    assert f(*args(K=60)) == _lib.KR_ERR_NUMEL_MOD8
    assert f(*args(lda_k=2)) == _lib.KR_ERR_LAYOUT
    assert f(*args(C=FAKE + 8)) == _lib.KR_ERR_ALIGNMENT
    assert f(*args(M=0)) == 0                                 # nothing to compute, nothing launched
    g = lib.kr_stream_wait_value32
    assert g(None, 1, 0, None, None) == _lib.KR_ERR_NULL_POINTER
    assert g(FAKE + 2, 1, 0, None, None) == _lib.KR_ERR_ALIGNMENT
    assert g(FAKE, 1, 0, FAKE + 1, None) == _lib.KR_ERR_ALIGNMENT
    assert g(FAKE, 1, -5, None, None) == _lib.KR_ERR_BAD_DIM
    k = lib.kr_flag_arrive_wait
    assert k(None, 8, 32, 0, None, None) == _lib.KR_ERR_NULL_POINTER
    assert k(FAKE, 0, 32, 0, None, None) == _lib.KR_ERR_BAD_DIM
    assert k(FAKE, 8, 30, 0, None, None) == _lib.KR_ERR_STRIPE          # consumers per producer must be whole
    assert k(FAKE + 2, 8, 32, 0, None, None) == _lib.KR_ERR_ALIGNMENT
    h = lib.kr_copy_engine_memcpy
    assert h(FAKE, FAKE + 64, -1, None) == _lib.KR_ERR_BAD_DIM
    assert h(None, None, 0, None) == 0                        # nothing to copy
    assert h(None, FAKE, 16, None) == _lib.KR_ERR_NULL_POINTER
    assert h(FAKE, None, 16, None) == _lib.KR_ERR_NULL_POINTER


def test_gemm_workspace_entries(lib):
    assert lib.kr_gemm_workspace_bytes(0, 128, 128) == 0
    assert lib.kr_gemm_workspace_bytes(8192, 8192, 8192) == 0
    need = lib.kr_gemm_workspace_bytes(128, 6656, 4096)
    assert need >= 2 * 128 * 6656 * 4 and need % (128 * 6656 * 4) == 0   # S fp32 partial products
    f = lib.kr_gemm_reduce_ws_bf16
    base = (FAKE, 4096, 1, FAKE, 6656, 1, 128, 6656, 4096, None, 0, 0, None, 0, 128, None, FAKE, 0, 0)
    assert f(*base, FAKE + 8, need, None) == _lib.KR_ERR_ALIGNMENT     # workspace not 16-byte aligned
    assert f(FAKE, 4096, 2, *base[3:], FAKE, need, None) == _lib.KR_ERR_LAYOUT
    g = lib.kr_gemm_reduce_ptrs_ws_bf16
    assert g(FAKE, 4096, 1, FAKE, 6656, 1, 128, 6656, 4096, None, 2, None, 0, 128, None, FAKE, 0, 0,
             FAKE, need, None) == _lib.KR_ERR_NULL_POINTER


def test_gemm_noalloc_entry_checks_arguments_first(lib, monkeypatch):
    """The allocation-free form validates like the others (nothing is looked up or launched for
    a rejected call) and refuses a split that its static scratch cannot hold."""
    f = lib.kr_gemm_reduce_noalloc_bf16
    base = (FAKE, 4096, 1, FAKE, 6656, 1, 128, 6656, 4096, None, 0, 0, None, 0, 128, None, FAKE, 0, 0)
    assert f(FAKE, 4096, 2, *base[3:], None) == _lib.KR_ERR_LAYOUT
    assert f(None, *base[1:], None) == _lib.KR_ERR_NULL_POINTER
    assert f(FAKE + 4, *base[1:], None) == _lib.KR_ERR_ALIGNMENT
    assert f(*base[:6], 0, 6656, 4096, None, 0, 0, None, 0, 0, None, FAKE, 0, 0, None) == 0   # M == 0: nothing to do
    monkeypatch.setenv("KRAKEN_AMD_GEMM_TILE", "128")
    monkeypatch.setenv("KRAKEN_AMD_GEMM_SPLITK", "16")                  # 16 partial products of 1024 x 2048 fp32
    assert lib.kr_gemm_workspace_bytes(1024, 2048, 4096) == 16 * 1024 * 2048 * 4 > (64 << 20)
    assert f(FAKE, 4096, 1, FAKE, 2048, 1, 1024, 2048, 4096, None, 0, 0, None, 0, 1024, None, FAKE, 0, 0,
             None) == _lib.KR_ERR_SCRATCH
    # an oversize shape with a bad argument reports the argument, as every other entry point would
    assert f(None, 4096, 1, FAKE, 2048, 1, 1024, 2048, 4096, None, 0, 0, None, 0, 1024, None, FAKE, 0, 0,
             None) == _lib.KR_ERR_NULL_POINTER
    assert f(FAKE + 2, 4096, 1, FAKE, 2048, 1, 1024, 2048, 4096, None, 0, 0, None, 0, 1024, None, FAKE, 0, 0,
             None) == _lib.KR_ERR_ALIGNMENT
    assert f(FAKE, 4096, 2, FAKE, 2048, 1, 1024, 2048, 4096, None, 0, 0, None, 0, 1024, None, FAKE, 0, 0,
             None) == _lib.KR_ERR_LAYOUT
    assert "scratch" in _lib.strerror(_lib.KR_ERR_SCRATCH)


def test_gemm_plan_reports_the_dispatch(lib, monkeypatch):
    """kr_gemm_plan names the kernel a shape gets, by the rule the launch itself uses."""
    p = _lib.gemm_plan(8192, 8192, 3584, False, 7, 1024, False, True)        # GEMM + reduce-scatter shape
    assert p["kernel"] == "gemm_dtl16_kernel" and p["tile"] == 256 and p["mfma"] == "16x16x32" and p["peers_on_mfma"]
    p = _lib.gemm_plan(4096, 8192, 1024, False, 7, 4096, True, False)        # every tile streams peers
    assert p["kernel"] == "gemm_dtl16_kernel" and p["mfma"] == "16x16x32" and p["peers_on_mfma"] and p["group_n"] == 16
    p = _lib.gemm_plan(8192, 3584, 8192, True)                               # all-gather matmul shape: 448 tiles of 256 columns
    assert p["kernel"] == "gemm_dtl16n7_kernel" and p["tile_n"] == 224 and p["group_n"] == 4 and p["tail_tiles"] == 0   # 512 of 224
    assert _lib.gemm_plan(8192, 3584, 8192, False)["tile_n"] == 256          # row-major B: no 224-column form
    assert _lib.gemm_plan(8192, 3584, 8192, True, 7, 8192)["tile_n"] == 256  # peers: not a plain product
    assert _lib.gemm_plan(8192, 3584, 8192, True, has_bias=True)["tile_n"] == 256
    assert _lib.gemm_plan(8192, 7168, 4096, True)["tile_n"] == 224           # 896 tiles = 3.5 rounds against 1024 = 4 rounds of 224
    assert _lib.gemm_plan(8192, 14336, 4096, True)["tile_n"] == 256          # 1792 tiles = 7 whole rounds already
    assert _lib.gemm_plan(8192, 4096, 8192, True)["tile_n"] == 256           # 224 does not divide N
    p = _lib.gemm_plan(256, 256, 100 * 8, False)                             # K not a multiple of 64
    assert p["kernel"] == "gemm_reduce_kernel" and p["tile"] == 128 and p["k_splits"] == 1
    need = lib.kr_gemm_workspace_bytes(128, 6656, 4096)
    p = _lib.gemm_plan(128, 6656, 4096, False, workspace_bytes=need)         # few tiles: split K loop
    assert p["tile"] == 128 and p["k_splits"] > 1
    assert _lib.gemm_plan(128, 6656, 4096, False)["k_splits"] == 1           # no workspace, no split
    p = _lib.gemm_plan(4352, 4096, 8192, False, workspace_bytes=1 << 30)     # 272 tiles: 16 tail tiles split
    assert p["tile"] == 256 and p["tail_tiles"] == 16 and p["tail_splits"] == 8
    assert _lib.gemm_plan(300, 8192 + 8, 4096, False)["ragged"]
    plan = (ctypes.c_int32 * 8)()
    assert lib.kr_gemm_plan(0, 64, 64, 0, 0, 0, 0, 0, 0, plan) == _lib.KR_ERR_BAD_DIM
    assert lib.kr_gemm_plan(64, 64, 64, 0, 16, 0, 0, 0, 0, plan) == _lib.KR_ERR_WORLD_SIZE
    assert lib.kr_gemm_plan(64, 64, 64, 0, 0, 65, 0, 0, 0, plan) == _lib.KR_ERR_BAND
    assert lib.kr_gemm_plan(64, 64, 64, 0, 0, 0, 0, 0, 0, None) == _lib.KR_ERR_NULL_POINTER
    monkeypatch.setenv("KRAKEN_AMD_GEMM_MFMA", "32")
    _lib.reload_env()
    try:
        assert _lib.gemm_plan(8192, 4096, 8192, True)["kernel"] == "gemm_dtl_kernel"
    finally:
        monkeypatch.delenv("KRAKEN_AMD_GEMM_MFMA")
        _lib.reload_env()


def test_split_fp32_argument_errors(lib):
    f = lib.kr_split_fp32
    assert f(FAKE, 16, 12, 12, 1, 0, FAKE, 36, None) == _lib.KR_ERR_NUMEL_MOD8
    assert f(None, 16, 16, 16, 1, 0, FAKE, 48, None) == _lib.KR_ERR_NULL_POINTER
    assert f(FAKE, 16, 16, 8, 1, 0, FAKE, 48, None) == _lib.KR_ERR_LAYOUT          # row stride shorter than the row
    assert f(FAKE, 16, 16, 16, 1, 0, FAKE, 40, None) == _lib.KR_ERR_LAYOUT         # side by side needs 3 * cols
    assert f(FAKE + 4, 16, 16, 16, 1, 0, FAKE, 48, None) == _lib.KR_ERR_ALIGNMENT
    assert f(FAKE, 16, 16, 18, 1, 0, FAKE, 48, None) == _lib.KR_ERR_ALIGNMENT      # fp32 rows not 16-byte aligned
    assert f(FAKE, 16, 16, 16, 1, 2, FAKE, 48, None) == _lib.KR_ERR_BAD_DIM
    assert f(None, 0, 16, 16, 1, 0, None, 48, None) == 0


def test_fp8_cast_argument_errors(lib):
    for f in (lib.kr_cast_fp8_to_bf16, lib.kr_cast_f32_to_fp8):
        assert f(FAKE, 24, FAKE, None) == _lib.KR_ERR_NUMEL_MOD8
        assert f(FAKE, -16, FAKE, None) == _lib.KR_ERR_BAD_DIM
        assert f(None, 32, FAKE, None) == _lib.KR_ERR_NULL_POINTER
        assert f(FAKE, 32, None, None) == _lib.KR_ERR_NULL_POINTER
        assert f(FAKE + 4, 32, FAKE, None) == _lib.KR_ERR_ALIGNMENT
        assert f(None, 0, None, None) == 0


def test_gemm_fp8_argument_errors(lib):
    f = lib.kr_gemm_fp8
    ok = (FAKE, 512, FAKE, 512, 256, 256, 512, FAKE, 2, None)
    def call(**kw):
        names = ("A", "lda", "Bt", "ldb", "M", "N", "K", "out", "kind", "stream")
        args = dict(zip(names, ok)); args.update(kw)
        return f(*[args[n] for n in names])
    assert call(M=128) == _lib.KR_ERR_BAD_DIM            # whole 256 x 256 tiles only
    assert call(N=384) == _lib.KR_ERR_BAD_DIM
    assert call(K=192, lda=192, ldb=192) == _lib.KR_ERR_BAD_DIM
    assert call(kind=3) == _lib.KR_ERR_BAD_DIM
    assert call(M=-256) == _lib.KR_ERR_BAD_DIM
    assert call(A=None) == _lib.KR_ERR_NULL_POINTER
    assert call(out=None) == _lib.KR_ERR_NULL_POINTER
    assert call(lda=256) == _lib.KR_ERR_LAYOUT           # rows shorter than K
    assert call(ldb=520) == _lib.KR_ERR_ALIGNMENT        # row stride not a multiple of 16 bytes
    assert call(Bt=FAKE + 8) == _lib.KR_ERR_ALIGNMENT
    assert call(M=0, A=None, Bt=None, out=None) == 0     # nothing to do, nothing launched
    g = lib.kr_all_gather_matmul_fp8
    base = dict(A=FAKE, lda=512, A_local=FAKE, lda_local=512, Bt=FAKE, ldb=512, M=2048, N=256, K=512, W=8, rank=3, splits=1,
                progress=FAKE, limit=0, status=None, out=FAKE, kind=2, stream=None)
    def gcall(**kw):
        args = dict(base); args.update(kw)
        return g(*args.values())
    assert gcall(W=0) == _lib.KR_ERR_WORLD_SIZE
    assert gcall(rank=8) == _lib.KR_ERR_STRIPE
    assert gcall(splits=3) == _lib.KR_ERR_BAND           # 2048 rows in 24 chunks
    assert gcall(lda_local=520) == _lib.KR_ERR_ALIGNMENT
    assert gcall(lda_local=256) == _lib.KR_ERR_LAYOUT
    assert gcall(progress=FAKE + 2) == _lib.KR_ERR_ALIGNMENT
    assert gcall(M=1024, N=384) == _lib.KR_ERR_BAD_DIM   # the product's own shape rule


def test_probe_argument_errors(lib):
    assert lib.kr_probe_read(FAKE, 24, None, None) == _lib.KR_ERR_NUMEL_MOD8
    assert lib.kr_probe_read(None, 32, None, None) == _lib.KR_ERR_NULL_POINTER
    assert lib.kr_probe_read(FAKE + 4, 32, None, None) == _lib.KR_ERR_ALIGNMENT
    assert lib.kr_probe_read(None, 0, None, None) == 0
    assert lib.kr_probe_copy(FAKE, None, 32, None) == _lib.KR_ERR_NULL_POINTER
    assert lib.kr_probe_copy(FAKE, FAKE + 8, 32, None) == _lib.KR_ERR_ALIGNMENT
    assert lib.kr_probe_copy(None, None, 0, None) == 0


def test_striped_share_numel(lib):
    f = lib.kr_striped_share_numel
    numel, W, block = 8 * 37, 4, 16
    shares = [f(numel, W, block, r) for r in range(W)]
    assert sum(shares) == numel
    from oracle import oracle as orc
    assert shares == [orc.striped_indices(numel, W, block, r).numel() for r in range(W)]
    assert f(numel, W, 12, 0) == _lib.KR_ERR_STRIPE
    assert f(numel, W, 16, 4) == _lib.KR_ERR_STRIPE
    assert f(numel + 4, W, 16, 0) == _lib.KR_ERR_NUMEL_MOD8


def test_rotated_argument_errors(lib):
    f = lib.kr_reduce_rotated_bf16
    assert f(FAKE, 4, 3, 16, 4, 1, FAKE, None) == _lib.KR_ERR_STRIPE
    assert f(FAKE, 4, 3, 12, 0, 1, FAKE, None) == _lib.KR_ERR_NUMEL_MOD8
    assert f(None, 4, 3, 16, 0, 1, FAKE, None) == _lib.KR_ERR_NULL_POINTER


def test_check_maps_codes_to_reference_exceptions():
    with pytest.raises(AssertionError, match="128-bit"):
        _lib.check(_lib.KR_ERR_NUMEL_MOD8, "x")
    with pytest.raises(ValueError):
        _lib.check(_lib.KR_ERR_LAYOUT, "x")
    with pytest.raises(_lib.KrakenAmdError):
        _lib.check(1, "x")
    _lib.check(0, "x")


def test_public_names_match_reference_layout():
    # kraken/comm/__init__.py:12-17, kraken/fused/__init__.py:17-27
    assert set(comm.__all__) == {"_copy_engine_all_gather_w_progress", "all_gather_w_progress",
                                 "one_shot_all_reduce", "two_shot_all_reduce"}
    assert set(fused.__all__) == {
        "all_gather_matmul", "gemm_one_shot_all_reduce_fused", "gemm_reduce_scatter",
        "gemm_reduce_scatter_ce_persistent", "one_shot_all_reduce_bias",
        "one_shot_all_reduce_bias_rms_norm", "rms_norm", "two_shot_all_reduce_bias",
        "two_shot_all_reduce_bias_rms_norm",
    }
    assert kraken_amd.__all__ == ["_lib", "_logging", "comm", "fused"]
    # kraken/_logging/__init__.py:1-4 (the PTX dump helper has no counterpart: nothing is compiled at run time)
    from kraken_amd import _logging
    assert set(_logging.__all__) == {"benchmark_with_event", "benchmark_with_profiler", "plot_experiment_comparison"}


def test_plot_experiment_comparison_writes_the_chart(tmp_path):
    from kraken_amd._logging import plot_experiment_comparison
    out = tmp_path / "sweep.png"
    plot_experiment_comparison(["(1, 5k)", "(2, 5k)", "(4, 5k)"], ["hip", "torch"], [[6.3, 14.6], [6.3, 13.4], [6.4, 13.6]],
                               str(out))
    assert out.stat().st_size > 1000 and out.read_bytes()[:4] == b"\x89PNG"
    with pytest.raises(AssertionError):
        plot_experiment_comparison(["a"], ["x", "y"], [[1.0]], str(out))      # a row per size, a value per experiment


def test_wrappers_assert_like_the_reference_and_refuse_host_tensors():
    s32 = torch.zeros(8, 4, 64, dtype=torch.float32)
    with pytest.raises(AssertionError, match="bfloat16"):
        comm.one_shot_all_reduce(s32)                       # one_shot_all_reduce.py:79
    with pytest.raises(AssertionError, match="128-bit"):
        comm.one_shot_all_reduce(torch.zeros(8, 3, 4, dtype=BF16))   # :80
    with pytest.raises(AssertionError):
        comm.two_shot_all_reduce(torch.zeros(3, 8, 64, dtype=BF16), BLOCK_SIZE=2048)  # BLOCK % W
    s = torch.zeros(8, 4, 64, dtype=BF16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        comm.one_shot_all_reduce(s)
    y = torch.empty(4, 64, dtype=BF16)
    w = torch.ones(64, dtype=BF16)
    with pytest.raises(AssertionError):
        fused.one_shot_all_reduce_bias_rms_norm(s, None, None, torch.ones(32, dtype=BF16), y)  # w.shape == (D,)
    with pytest.raises(AssertionError):
        fused.two_shot_all_reduce_bias_rms_norm(torch.zeros(8, 1, 72, dtype=BF16), None, None,
                                                torch.ones(72, dtype=BF16), torch.empty(1, 72, dtype=BF16))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fused.one_shot_all_reduce_bias_rms_norm(s, None, None, w, y)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fused.rms_norm(torch.zeros(4, 64, dtype=BF16), w)
    a, b = torch.zeros(64, 32, dtype=BF16), torch.zeros(32, 64, dtype=BF16)
    with pytest.raises(AssertionError, match="Inner dimensions"):
        fused.gemm_one_shot_all_reduce_fused(a, torch.zeros(16, 64, dtype=BF16))
    with pytest.raises(AssertionError, match="divisible by world_size"):
        fused.gemm_reduce_scatter(torch.zeros(66, 32, dtype=BF16), b, world_size=4)
    with pytest.raises(ValueError, match="b.T must be contiguous"):
        fused.all_gather_matmul(torch.zeros(4, 16, 32, dtype=BF16), b)   # all_gather_matmul.py:158-160
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fused.gemm_one_shot_all_reduce_fused(a, b)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libkraken_amd.so")
    with pytest.raises(RuntimeError, match="kraken_amd.build"):
        _lib.load()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one rank on one GPU: any other --gpus value ends with a message and exit status 2
    before anything touches a device."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, str(Path(__file__).resolve().parents[1] / "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "--gpus 2 is not supported" in r.stderr and r.stdout == ""
