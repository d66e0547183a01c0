"""Build libduq_hip.so in-tree with hipcc for gfx950: ``python -m duqlinear4bitcuda_amd.build``."""
from __future__ import annotations

import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(clean: bool = True, jobs: int = 8, verbose: bool = False) -> str:
    csrc = os.path.join(_HERE, "csrc")
    if clean:
        subprocess.run(["make", "-C", csrc, "clean"], check=True, capture_output=not verbose)
    res = subprocess.run(["make", "-C", csrc, f"-j{jobs}"], capture_output=not verbose, text=True)
    if res.returncode != 0:
        sys.stderr.write((res.stdout or "") + (res.stderr or ""))
        raise RuntimeError("hipcc build of libduq_hip.so failed")
    return os.path.join(_HERE, "libduq_hip.so")


if __name__ == "__main__":
    print(build(verbose=True))
