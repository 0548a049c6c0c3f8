"""Compiles libmi355_moe.so for gfx950 with hipcc (python -m therock_amd.build)."""
from __future__ import annotations

import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(force: bool = True, jobs: int = 4, verbose: bool = False) -> str:
    """Runs the csrc Makefile.  force=True recompiles every object."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), f"-j{jobs}"]
    if force:
        cmd.append("-B")
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        sys.stdout.write(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libmi355_moe.so failed")
    return os.path.join(_HERE, "libmi355_moe.so")


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
