"""Compile oracle/oracle_c.c into oracle/_build/liboracle_c.so with gcc (test infrastructure).

The reference is pure Python/Triton with no C/C++ sources, so there is nothing
to compile into oracle/_ref/.
"""
from __future__ import annotations

import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT = HERE / "_build" / "liboracle_c.so"


def build(verbose: bool = True) -> Path:
    OUT.parent.mkdir(exist_ok=True)
    # -ffp-contract=off: no fused multiply-add, the loops must round like the fp32 formulas
    cmd = ["gcc", "-O2", "-ffp-contract=off", "-shared", "-fPIC", str(HERE / "oracle_c.c"), "-lm", "-o", str(OUT)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"gcc failed:\n{proc.stdout}\n{proc.stderr}")
    if verbose:
        print(f"built {OUT}")
    return OUT


if __name__ == "__main__":
    build()
