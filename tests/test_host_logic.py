"""Host-side helpers that need no GPU."""

import torch.nn as nn


def test_merge_joins_adjacent_ranges_only():
    from yafsdp_amd.optim import _merge

    assert _merge([]) == []
    assert _merge([(5, 9), (0, 5), (9, 9), (12, 20)]) == [(0, 9), (12, 20)]
    assert _merge([(3, 3)]) == []
    assert _merge([(0, 4), (6, 8), (4, 6)]) == [(0, 8)]


def test_root_modules_of_a_list():
    from yafsdp_amd.fully_shard import _get_root_modules

    a = nn.Sequential(nn.Linear(2, 2), nn.Linear(2, 2))
    b = nn.Linear(2, 2)
    assert _get_root_modules([a, b]) == [a, b]
    assert _get_root_modules([a[0], a, b, a[1]]) == [a, b]  # members of `a` are dropped
    assert _get_root_modules([b, b]) == [b]


def test_param_names_of_a_module_list():
    from yafsdp_amd.fully_shard import _param_names

    a, b = nn.Linear(2, 2), nn.Linear(2, 2, bias=False)
    assert _param_names((a,), list(a.parameters())) == ["weight", "bias"]
    assert _param_names((a, b), [b.weight, a.bias]) == ["1.weight", "0.bias"]


def test_flat_adamw_rejects_bad_hyperparameters():
    import pytest
    import torch

    from yafsdp_amd.optim import FlatAdamW

    p = [nn.Parameter(torch.zeros(4))]
    for kw in (dict(lr=-1.0), dict(eps=-1e-8), dict(betas=(1.0, 0.9)), dict(weight_decay=-0.1)):
        with pytest.raises(ValueError):
            FlatAdamW(p, **kw)
    opt = FlatAdamW(p, lr=1e-3)  # construction needs no GPU; stepping a CPU parameter does
    p[0].grad = torch.zeros(4)
    with pytest.raises(TypeError):
        opt.step()


def test_sizes_to_slices_docstring_example():
    """The one worked example the reference holds for this path (ya_fsdp/_collectives.py:79-90)."""
    from yafsdp_amd._collectives import sizes_to_slices

    assert sizes_to_slices([20, 20, 30]) == [slice(0, 20, None), slice(20, 40, None), slice(40, 70, None)]
    assert sizes_to_slices([]) == []
    assert sizes_to_slices([0, 3, 0]) == [slice(0, 0), slice(0, 3), slice(3, 3)]


def test_staging_slot_state_machine_against_a_simulated_runtime():
    """``yafsdp_amd/csrc/stage_ring.h`` (the slots that carry per-call pointer arrays to the table kernels) driven by
    a simulated runtime on the host: random streams, repeated and fresh tensor sets, failed copies and launches,
    partial completion; every kernel must be ordered behind the copy it reads and no copy may overtake a queued
    reader (tests/c/stage_ring_check.cpp)."""
    import importlib.util
    import os
    import subprocess

    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c")
    spec = importlib.util.spec_from_file_location("c_build", os.path.join(here, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    binary = mod.build_stage_ring_check()
    r = subprocess.run([binary], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip().endswith("PASS"), r.stdout[-2000:] + r.stderr[-2000:]


def _run_bench(*flags):
    import subprocess
    import sys
    from pathlib import Path

    bench = Path(__file__).resolve().parents[1] / "bench.py"
    return subprocess.run([sys.executable, str(bench), *flags], capture_output=True, text=True, timeout=300)


def test_bench_refuses_more_than_one_gpu():
    """Every figure of this build is one GPU's: a request for more ends at once, with a message that says so and
    without a result line on stdout."""
    done = _run_bench("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert done.returncode != 0
    assert "ONE GPU" in done.stderr + done.stdout
    assert "{" not in done.stdout


def test_bench_has_no_cpu_path_to_measure():
    """Without a GPU the benchmark must not fall back to anything that runs on the host."""
    import torch

    if torch.cuda.is_available():
        import pytest

        pytest.skip("a GPU is visible")
    done = _run_bench("--steps", "1", "--warmup", "0")
    assert done.returncode != 0
    assert "no GPU" in done.stderr + done.stdout
    assert "{" not in done.stdout
