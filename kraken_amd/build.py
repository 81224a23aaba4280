"""Build libkraken_amd.so (gfx950) from kraken_amd/csrc/*.hip with hipcc.

    python -m kraken_amd.build            # compile + link, in-tree

hipcc cross-compiles without a GPU.  Objects go to kraken_amd/lib/obj/, the
shared library to kraken_amd/lib/libkraken_amd.so.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libkraken_amd.so"
ARCH = "gfx950"

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",
    # the k-steps of the GEMM kernels are fully unrolled by "#pragma unroll"; above the default limit
    # (16384 instructions) the request is dropped without a word and register arrays turn into scratch
    "-mllvm", "-pragma-unroll-threshold=1048576",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(hipcc: str, src: Path, obj: Path) -> None:
    cmd = [hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stdout}\n{proc.stderr}")


def build(verbose: bool = True) -> Path:
    hipcc = hipcc_path()
    obj_dir = LIB_DIR / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    objs = [obj_dir / (s.stem + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        list(pool.map(lambda so: _compile(hipcc, *so), zip(srcs, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {[s.name for s in srcs]}")
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
