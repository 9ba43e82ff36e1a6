"""The C ABI used from plain C: ``tests/c/abi_check`` (no Python, no torch in
the process) runs gather-in, bound scatter-out, the two launches that do the
work of two each, post-reduce, gradient norm, clip coefficient and the fused
AdamW step on device buffers it allocates with the HIP runtime and compares
each with the C oracle."""

import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "c", "abi_check")


@pytest.mark.gpu
def test_plain_c_program_passes():
    if not os.path.exists(BIN):
        pytest.fail(f"{BIN} is not built: run `python tests/c/build.py` (the build entry point does)")
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert r.stdout.strip().endswith("PASS")
    assert r.stdout.count("\nok ") >= 18


def test_c_program_source_uses_only_the_public_header():
    src = open(os.path.join(HERE, "c", "abi_check.c")).read()
    assert '#include "../../include/yafsdp_hip.h"' in src
    assert "torch" not in src.replace("no torch", "")
