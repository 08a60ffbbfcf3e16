"""Build libexo_mi355x.so (gfx950) from exo_amd/csrc/*.hip with hipcc.

Usage: ``python -m exo_amd.build`` (also called by ``__graft_entry__.build()``).
The library is written next to this file; object files go to ``build/``.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "libexo_mi355x.so"
SOURCES = ["quant.hip", "qmv.hip", "qmv_mfma.hip", "qmv_quad.hip", "qmv_w16.hip", "qmm.hip", "sdpa.hip", "sdpa_prefill.hip", "elementwise.hip", "kvwire.hip", "sampling.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd: list[str]) -> None:
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(
        ln for ln in r.stderr.splitlines() if "not a recognized feature" not in ln
    )
    if r.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{r.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(verbose: bool = True, extra_flags: list[str] | None = None) -> Path:
    objdir = PKG.parent / "build" / "obj"
    objdir.mkdir(parents=True, exist_ok=True)
    flags = FLAGS + (extra_flags or [])

    def compile_one(src: str) -> str:
        obj = objdir / (Path(src).stem + ".o")
        _run([HIPCC, *flags, "-c", str(CSRC / src), "-o", str(obj)])
        if verbose:
            print(f"[exo_amd.build] compiled {src}", flush=True)
        return str(obj)

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *objs])
    if verbose:
        print(f"[exo_amd.build] linked {LIB}", flush=True)
    return LIB


if __name__ == "__main__":
    build()
