"""Build the plain-C restatement (``bufpath_ref.c``) into ``libbufpath_ref.so``.

Test infrastructure only.  ``-ffp-contract=off`` and no fast-math so that every
binary32 operation rounds exactly once, as the torch ops it restates do.
"""

from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "bufpath_ref.c")
OUT = os.path.join(HERE, "libbufpath_ref.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(OUT) and os.path.getmtime(OUT) >= os.path.getmtime(SRC):
        return OUT
    cmd = [
        "gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off",
        "-fno-fast-math", "-Wall", "-Wextra", "-o", OUT, SRC, "-lm",
    ]
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    print(build())
