"""Builds ``tests/c/abi_check`` (plain C on the C ABI of libyafsdp_hip.so, checked
against the C oracle) with gcc.  Test infrastructure; run from anywhere:
``python tests/c/build.py``.  Needs both libraries built first."""

from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "abi_check")
SRC = os.path.join(HERE, "abi_check.c")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def build() -> str:
    for lib in (os.path.join(ROOT, "yafsdp_amd", "libyafsdp_hip.so"), os.path.join(ROOT, "oracle", "libbufpath_ref.so")):
        if not os.path.exists(lib):
            raise RuntimeError(f"{lib} is missing: build it first")
    cmd = [
        "gcc", "-O2", "-std=c11", "-Wall", "-D__HIP_PLATFORM_AMD__", f"-I{ROCM}/include", SRC, "-o", OUT,
        f"-L{ROOT}/yafsdp_amd", f"-L{ROOT}/oracle", f"-L{ROCM}/lib", "-lyafsdp_hip", "-lbufpath_ref", "-lamdhip64", "-lm",
        f"-Wl,-rpath,$ORIGIN/../../yafsdp_amd:$ORIGIN/../../oracle:{ROCM}/lib",
    ]
    subprocess.run(cmd, check=True)
    return OUT


RING_OUT = os.path.join(HERE, "stage_ring_check")


def build_stage_ring_check() -> str:
    """Host-only simulation of the staging slots' state machine (``yafsdp_amd/csrc/stage_ring.h``): g++, no HIP."""
    cmd = ["g++", "-O1", "-std=c++17", "-Wall", os.path.join(HERE, "stage_ring_check.cpp"), "-o", RING_OUT]
    subprocess.run(cmd, check=True)
    return RING_OUT


if __name__ == "__main__":
    print(build())
    print(build_stage_ring_check())
