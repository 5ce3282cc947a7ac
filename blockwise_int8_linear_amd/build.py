"""Builds libbi8.so in-tree with hipcc for gfx950:  python -m blockwise_int8_linear_amd.build [--clean]"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")


def build(force: bool = False, jobs: int = 8, quiet: bool = True) -> str:
    cmd = ["make", "-C", CSRC, f"-j{jobs}"] + (["-B"] if force else [])
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0 or not quiet:
        # hipcc's host pass prints a harmless note about the packed-fp32 feature flag
        print("\n".join(l for l in res.stdout.splitlines() if "not a recognized feature" not in l))
    if res.returncode != 0:
        raise RuntimeError("building libbi8.so failed")
    return os.path.join(HERE, "libbi8.so")


if __name__ == "__main__":
    if "--clean" in sys.argv:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True)
    print(build(force="--force" in sys.argv, quiet=False))
