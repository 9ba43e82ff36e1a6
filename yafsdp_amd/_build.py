"""Build ``libyafsdp_hip.so`` (gfx950 kernels + C ABI) in-tree with hipcc.

Usage: ``python -m yafsdp_amd._build``.  The library is built next to this file
so that it travels with the source tree; nothing is installed elsewhere.
"""

from __future__ import annotations

import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libyafsdp_hip.so")
SOURCES = ["api.hip", "flat.hip", "gather.hip", "scatter.hip", "optim.hip", "fan.hip", "postsumsq.hip", "fused.hip"]
HEADERS = ["elem.hip.h", "flat_kernels.hip.h", "table_kernels.hip.h", "optim_kernels.hip.h", "fan_kernels.hip.h",
           "post_sumsq_kernels.hip.h", "fused_kernels.hip.h", "launch.h", "stage_ring.h", "tuning.h"]
ARCH = "gfx950"

# -ffp-contract=off: every multiply and add of the path rounds on its own, as
# the separate torch ops of the reference do.  packed-fp32 ops are disabled
# for all device code of this library.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src: str, obj: str) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        print(err)


def build(force: bool = True, jobs: int = 8) -> str:
    """Compile every translation unit and link the shared library."""
    srcs = [os.path.join(CSRC, s) for s in SOURCES + HEADERS] + [os.path.join(HERE, "..", "include", "yafsdp_hip.h")]
    if not force and os.path.exists(OUT) and all(os.path.getmtime(OUT) >= os.path.getmtime(s) for s in srcs):
        return OUT
    build_dir = os.path.join(HERE, "build")
    os.makedirs(build_dir, exist_ok=True)
    objs = [os.path.join(build_dir, s.replace(".hip", ".o")) for s in SOURCES]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(_compile, SOURCES, objs))
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", OUT, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return OUT


CEILINGS_OUT = os.path.join(HERE, "libyafsdp_ceilings.so")


def build_ceilings(force: bool = True) -> str:
    """Compile the measurement-only stream-mix mover (``csrc/ceilings.hip``) into a library of its own; only the
    benchmark's hbm-ceilings workload loads it."""
    src = os.path.join(CSRC, "ceilings.hip")
    if not force and os.path.exists(CEILINGS_OUT) and os.path.getmtime(CEILINGS_OUT) >= os.path.getmtime(src):
        return CEILINGS_OUT
    cmd = [_hipcc(), *HIPCC_FLAGS, "-shared", src, "-o", CEILINGS_OUT]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        noise = "is not a recognized feature for this target"
        raise RuntimeError("hipcc failed on ceilings.hip:\n" + "\n".join(l for l in r.stderr.splitlines() if noise not in l))
    return CEILINGS_OUT


TENSORLIST_SRC = os.path.join(CSRC, "tensorlist.cpp")
TENSORLIST_OUT = os.path.join(HERE, "_tensorlist.so")


def build_tensorlist(force: bool = True) -> str:
    """Compile the host-side tensor-list helper of the Python binding (plain C++ against the installed torch's
    headers; no device code)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    if not force and os.path.exists(TENSORLIST_OUT) and os.path.getmtime(TENSORLIST_OUT) >= os.path.getmtime(TENSORLIST_SRC):
        return TENSORLIST_OUT
    lib_dir = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [
        os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
        TENSORLIST_SRC, "-o", TENSORLIST_OUT,
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-DTORCH_API_INCLUDE_EXTENSION_H",
        *[f"-I{p}" for p in cpp_extension.include_paths()], f"-I{sysconfig.get_paths()['include']}",
        f"-L{lib_dir}", "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_python", f"-Wl,-rpath,{lib_dir}",
    ]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"compiling tensorlist.cpp failed:\n{r.stderr[-4000:]}")
    return TENSORLIST_OUT


if __name__ == "__main__":
    print(build())
    print(build_tensorlist())
    print(build_ceilings())
