"""Build the C part of the oracle: oracle/_build/libqmm_ref.so (gcc, OpenMP).

TEST INFRASTRUCTURE ONLY.  The reference itself has no C/C++ source on this path
(its arithmetic is in the un-vendored mlx wheel), so there is no ``oracle/_ref``
build of reference sources."""

from __future__ import annotations

import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIB = HERE / "_build" / "libqmm_ref.so"


def build(verbose: bool = True) -> Path:
    LIB.parent.mkdir(exist_ok=True)
    cmd = ["gcc", "-O3", "-mavx2", "-mfma", "-fopenmp", "-shared", "-fPIC", "-o", str(LIB),
           str(HERE / "qmm_ref.c")]
    subprocess.run(cmd, check=True)
    if verbose:
        print(f"[oracle.build] built {LIB}", flush=True)
    return LIB


if __name__ == "__main__":
    build()
