"""Builds trl_amd/lib/libtrlk.so with hipcc for gfx950 (`python trl_amd/build.py`: run as a script, because importing the package needs the library)."""
from __future__ import annotations

import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def build(clean: bool = True, jobs: int = 4) -> str:
    if clean:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", CSRC, f"-j{jobs}"], check=True)
    # the same device code under a sanitized host build: what tests/test_abi_sanitized.py loads
    subprocess.run(["make", "-C", CSRC, f"-j{jobs}", "asan"], check=True)
    out = os.path.join(os.path.dirname(CSRC), "lib", "libtrlk.so")
    if not os.path.exists(out):
        raise RuntimeError(f"build finished but {out} does not exist")
    return out


if __name__ == "__main__":
    print(build(clean="--no-clean" not in sys.argv))
