"""ctypes binding of libkraken_amd.so (the C ABI in include/kraken_amd.h)."""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libkraken_amd.so"

# negative return codes of the library (include/kraken_amd.h)
KR_OK = 0
KR_ERR_NULL_POINTER = -1
KR_ERR_ALIGNMENT = -2
KR_ERR_NUMEL_MOD8 = -3
KR_ERR_BAD_DIM = -4
KR_ERR_WORLD_SIZE = -5
KR_ERR_BIAS_SHAPE = -6
KR_ERR_ROW_TOO_LONG = -7
KR_ERR_BAND = -8
KR_ERR_LAYOUT = -9
KR_ERR_STRIPE = -10
KR_ERR_SCRATCH = -11

_SIGNATURES = {
    "kr_version": (c_int, []),
    "kr_init": (c_int, []),
    "kr_strerror": (c_char_p, [c_int]),
    "kr_reload_env": (None, []),
    "kr_reduce_bf16": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p],
    ),
    "kr_reduce_ptrs_bf16": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p],
    ),
    "kr_reduce_striped_ptrs_bf16": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_int64, c_int, c_void_p, c_void_p],
    ),
    "kr_reduce_rmsnorm_ptrs_bf16": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_void_p, c_float, c_void_p, c_void_p],
    ),
    "kr_gemm_reduce_ptrs_bf16": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p, c_int, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int64, c_void_p],
    ),
    "kr_reduce_striped_bf16": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int64, c_int, c_void_p, c_void_p],
    ),
    "kr_striped_share_numel": (c_int64, [c_int64, c_int, c_int64, c_int]),
    "kr_reduce_rmsnorm_bf16": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p, c_float, c_void_p, c_void_p],
    ),
    "kr_rmsnorm_workspace_bytes": (c_int64, [c_int, c_int64, c_int64]),
    "kr_reduce_rmsnorm_ws_bf16": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p, c_float, c_void_p,
         c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "kr_reduce_rmsnorm_ptrs_ws_bf16": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_void_p, c_float, c_void_p,
         c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "kr_rmsnorm_bf16": (c_int, [c_void_p, c_void_p, c_float, c_int64, c_int64, c_void_p, c_void_p]),
    "kr_gemm_reduce_bf16": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p, c_int, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int64, c_void_p],
    ),
    "kr_gemm_reduce_noalloc_bf16": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p, c_int, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int64, c_void_p],
    ),
    "kr_gemm_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64]),
    "kr_gemm_reduce_ws_bf16": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p, c_int, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int64,
         c_void_p, c_int64, c_void_p],
    ),
    "kr_gemm_reduce_ptrs_ws_bf16": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p, c_int, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int64,
         c_void_p, c_int64, c_void_p],
    ),
    "kr_all_gather_matmul_bf16": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p],
    ),
    "kr_stream_write_value32": (c_int, [c_void_p, ctypes.c_uint32, c_void_p]),
    "kr_gemm_producer_bf16": (
        c_int,
        [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p,
         c_int, c_int, c_void_p, c_void_p, c_void_p],
    ),
    "kr_stream_wait_value32": (c_int, [c_void_p, ctypes.c_uint32, c_int64, c_void_p, c_void_p]),
    "kr_copy_engine_memcpy": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "kr_flag_arrive_wait": (c_int, [c_void_p, c_int, c_int, c_int64, c_void_p, c_void_p]),
    "kr_reduce_rotated_bf16": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int, c_int, c_void_p, c_void_p]),
    "kr_split_fp32": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_int64, c_void_p]),
    "kr_cast_fp8_to_bf16": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "kr_cast_f32_to_fp8": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "kr_gemm_fp8": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p]),
    "kr_all_gather_matmul_fp8": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                         c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_int, c_void_p]),
    "kr_gemm_plan": (c_int, [c_int64, c_int64, c_int64, c_int, c_int, c_int64, c_int, c_int, c_int64, c_void_p]),
    "kr_probe_read": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "kr_probe_copy": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
}

EXPORTS = tuple(_SIGNATURES)

_lib = None


class KrakenAmdError(RuntimeError):
    """A HIP error reported by a kernel launch (positive return code)."""


def load() -> ctypes.CDLL:
    """Load libkraken_amd.so once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m kraken_amd.build` "
                "(kraken_amd has no CPU or PyTorch fallback)"
            )
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def gemm_plan(M: int, N: int, K: int, b_transposed: bool, n_peers: int = 0, band_rows: int | None = None,
              has_bias: bool = False, has_c_full: bool = False, workspace_bytes: int = 0) -> dict:
    """The kernel ``kr_gemm_reduce_*_bf16`` picks for a shape (``kr_gemm_plan``), as a dict with the
    kernel's name as a profiler lists it."""
    plan = (ctypes.c_int32 * 8)()
    rc = load().kr_gemm_plan(M, N, K, int(b_transposed), n_peers, M if band_rows is None else band_rows,
                             int(has_bias), int(has_c_full), workspace_bytes, plan)
    check(rc, "gemm_plan")
    tile, block, splits, tail, tail_splits, group_n, mfma_peers, ragged = list(plan)
    n224 = bool(ragged & 2)
    ragged &= 1
    if tile == 256:
        kernel = "gemm_dtl16n7_kernel" if n224 else "gemm_dtl16_kernel" if block == 16 else "gemm_dtl_kernel"
    else:
        kernel = "gemm_reduce_kernel"
    return {"kernel": kernel, "tile": tile, "mfma": "16x16x32" if block == 16 else "32x32x16", "k_splits": splits,
            "tail_tiles": tail, "tail_splits": tail_splits, "group_n": group_n, "peers_on_mfma": bool(mfma_peers),
            "ragged": bool(ragged), "tile_n": 224 if n224 else tile}


def reload_env() -> None:
    """Make the library read the KRAKEN_AMD_* environment switches again (it reads them once)."""
    load().kr_reload_env()


def strerror(code: int) -> str:
    return load().kr_strerror(int(code)).decode()


def check(code: int, what: str) -> None:
    """Map a library return code to the exception the reference would raise."""
    if code == KR_OK:
        return
    msg = f"{what}: {strerror(code)} (code {code})"
    if code > 0:
        raise KrakenAmdError(msg)
    if code in (KR_ERR_LAYOUT, KR_ERR_NULL_POINTER):
        raise ValueError(msg)
    raise AssertionError(msg)


def require_device(*tensors: torch.Tensor | None) -> torch.device:
    """All given tensors must live on one HIP device (no host fallback exists)."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "kraken_amd kernels run on a HIP device only; got a tensor on "
                f"'{t.device}' (there is no CPU fallback)"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    if dev is None:
        raise RuntimeError("no device tensor given")
    return dev


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def current_stream(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def copy_engine_copy(dst: torch.Tensor, src: torch.Tensor, stream: int) -> None:
    """``dst.copy_(src)`` on the copy engines (``kr_copy_engine_memcpy``): both contiguous,
    same dtype and number of elements, on the stream given (a raw ``hipStream_t``)."""
    assert dst.is_contiguous() and src.is_contiguous() and dst.dtype == src.dtype and dst.numel() == src.numel()
    rc = load().kr_copy_engine_memcpy(dst.data_ptr(), src.data_ptr(), src.numel() * src.element_size(), stream)
    check(rc, "copy_engine_memcpy")

