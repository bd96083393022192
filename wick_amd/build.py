"""Builds the gfx950 kernels + C ABI (hipcc cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_DIR = os.path.join(_HERE, "lib")


def build_library(force: bool = True, jobs: int = 8) -> str:
    """Compiles every HIP source for gfx950 into wick_amd/lib/libwick_rocm.{so,a}.

    ``force`` rebuilds even when the outputs are newer than the sources.
    Returns the path of the shared library."""
    cmd = ["make", "-C", CSRC, f"-j{jobs}"]
    if force:
        cmd.append("-B")
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building libwick_rocm failed:\n" + proc.stdout[-4000:])
    so = os.path.join(LIB_DIR, "libwick_rocm.so")
    if not os.path.exists(so):
        raise RuntimeError("build finished but " + so + " is missing")
    return so
