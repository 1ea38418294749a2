"""Builds libmta_hip.so in-tree:  python -m multitokenatention_triton_amd.build

hipcc cross-compiles for gfx950 without a GPU.  Packed-fp32 VALU forms are switched off
(-target-feature -packed-fp32-ops): the compiler would otherwise form v_pk_*_f32 from
ordinary float code.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def build(force: bool = True, jobs: int = 8) -> str:
    cmd = ["make", "-C", os.path.join(HERE, "csrc"), f"-j{jobs}"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    out = os.path.join(HERE, "libmta_hip.so")
    assert os.path.exists(out)
    return out


if __name__ == "__main__":
    print(build(force="--no-force" not in sys.argv))
