"""Builds libclusten_hip.so for gfx950 by driving `make` in csrc/ (hipcc cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB = os.path.join(_HERE, "lib", "libclusten_hip.so")


def build(jobs: int | None = None, clean: bool = False) -> str:
    """Compile every HIP translation unit and link the shared library; returns its path."""
    jobs = jobs or min(16, os.cpu_count() or 1)
    if clean:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True)
    subprocess.run(["make", "-C", CSRC, "-j%d" % jobs], check=True)
    if not os.path.exists(LIB):
        raise RuntimeError("make finished but %s is missing" % LIB)
    return LIB


if __name__ == "__main__":
    print(build())
