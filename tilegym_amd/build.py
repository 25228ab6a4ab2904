"""Build recipe for libtilegym_hip.so (hipcc, gfx950).  Cross-compiles without a GPU."""

from __future__ import annotations

import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libtilegym_hip.so")


def build(force: bool = True, jobs: int = 8, verbose: bool = False, check: bool = False) -> str:
    """Compile every HIP translation unit and link the shared library in-tree.

    ``force=True`` rebuilds all objects (``make -B``); returns the library path.  ``check=True`` also runs
    ``make check``: the kernels' assembly against the hardware rules around their inline-assembly loads
    (csrc/check_hazards.py; about half a minute more)."""
    cmd = ["make", "-C", CSRC, f"-j{int(jobs)}"]
    if force:
        cmd.append("-B")
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("hipcc build of libtilegym_hip.so failed (see output above)")
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"build finished but {LIB_PATH} is missing")
    if check:
        res = subprocess.run(["make", "-C", CSRC, "check"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if verbose or res.returncode != 0:
            print(res.stdout)
        if res.returncode != 0:
            raise RuntimeError("check_hazards.py reported findings on the built kernels (see output above)")
    return LIB_PATH


if __name__ == "__main__":
    import sys

    print(build(force=True, verbose=True, check="--check" in sys.argv[1:]))
