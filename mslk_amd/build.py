"""Builds mslk_amd/libmslk_amd.so with hipcc for gfx950:  python -m mslk_amd.build [--force]"""
from __future__ import annotations

import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(force: bool = False, jobs: int = 8) -> str:
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), f"-j{jobs}"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    return os.path.join(_HERE, "libmslk_amd.so")


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
