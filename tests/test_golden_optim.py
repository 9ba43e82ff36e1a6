"""Committed golden vectors of the optimizer-side passes and the reduce fan-in
(tests/golden/optim_small.npz, written by tests/golden/make_golden_optim.py).

CPU: the oracle still reproduces them.  GPU: the HIP path reproduces them
through the C ABI (the sum of squares to binary64 rounding: its order of
additions is the kernel's own)."""

import os

import numpy as np
import pytest
import torch

from oracle import cref, torch_ops
from tests.helpers import assert_bits_equal

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "optim_small.npz"),
               allow_pickle=False)
DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
ADAM_CASES = {
    "adamw_first": (True, 0.9, 0.1, 1, "bf16", None, False),
    "adamw_scaled": (True, 0.9, 0.1, 7, "f16", 0.37, True),
    "adam_l2": (False, 0.3, 0.01, 3, None, None, False),
}
FANIN_CASES = {"fanin_bf16": ("bf16", "f32", 8.0, True, 8), "fanin_f32": ("f32", "bf16", 3.0, False, 3)}
HP = dict(lr=3e-4, beta2=0.95, eps=1e-8)


def tens(key: str, name: str) -> torch.Tensor:
    a = GOLD[key]
    if name == "f32":
        return torch.from_numpy(a.view(np.int32).copy()).view(torch.float32)
    return torch.from_numpy(a.view(np.int16).copy()).view(DT[name])


def _impl(which):
    if which == "oracle":
        return None
    from yafsdp_amd import _native

    return _native


IMPLS = ["oracle", pytest.param("hip", marks=pytest.mark.gpu)]


@pytest.mark.parametrize("which", IMPLS)
@pytest.mark.parametrize("name", list(ADAM_CASES))
def test_adam_vectors(which, name):
    nat = _impl(which)
    decoupled, beta1, wd, step, out_name, gscale, zero = ADAM_CASES[name]
    dev = "cpu" if nat is None else "cuda:0"
    p, g, m, v = (tens(f"{name}_{k}_in", "f32").to(dev) for k in "pgmv")
    out16 = None if out_name is None else torch.zeros(p.numel(), dtype=DT[out_name], device=dev)
    kw = dict(lr=HP["lr"], beta1=beta1, beta2=HP["beta2"], eps=HP["eps"], weight_decay=wd, step=step,
              decoupled=decoupled, zero_grad=zero)
    if nat is None:
        cref.adamw_step(p, g, m, v, out16, grad_scale=gscale, **kw)
    else:
        gs = None if gscale is None else torch.tensor([gscale], device=dev)
        nat.adamw_step(p, g, m, v, out16, grad_scale=gs, **kw)
    for k, t in zip("pgmv", (p, g, m, v)):
        assert_bits_equal(t, tens(f"{name}_{k}_out", "f32"), f"{name} {k}")
    if out16 is not None:
        assert_bits_equal(out16, tens(f"{name}_out16", out_name), f"{name} out16")


@pytest.mark.parametrize("which", IMPLS)
@pytest.mark.parametrize("dt", list(DT))
def test_sumsq_and_scale_vectors(which, dt):
    nat = _impl(which)
    x = tens(f"sumsq_{dt}_in", dt)
    want = float(GOLD[f"sumsq_{dt}_out"][0])
    if nat is None:
        got = cref.sumsq(x)
        y = x.clone()
        cref.flat_scale(y, 0.7334219)
    else:
        d = x.to("cuda:0")
        out = torch.zeros(1, dtype=torch.float64, device="cuda:0")
        nat.flat_sumsq(d, out, nat.sumsq_workspace(torch.device("cuda:0")))
        got = out.item()
        y = d.clone()
        nat.flat_scale(y, torch.tensor([0.7334219], device="cuda:0"))
    assert abs(got - want) <= 1e-13 * want
    assert_bits_equal(y, tens(f"scale_{dt}_out", dt), "scale")


@pytest.mark.parametrize("which", IMPLS)
def test_clip_vectors(which):
    nat = _impl(which)
    for k in range(3):
        sumsq, max_norm = GOLD[f"clip_{k}"].tolist()
        want = GOLD[f"clip_{k}_out"]
        if nat is None:
            got = np.array(cref.clip_coef(sumsq, max_norm), dtype=np.float32)
        else:
            nc = torch.zeros(2, dtype=torch.float32, device="cuda:0")
            nat.clip_coef(torch.tensor([sumsq], dtype=torch.float64, device="cuda:0"), max_norm, nc)
            got = nc.cpu().numpy()
        assert got.view(np.uint32).tolist() == want.view(np.uint32).tolist(), (k, got, want)


@pytest.mark.parametrize("which", IMPLS)
@pytest.mark.parametrize("name", list(FANIN_CASES))
def test_fanin_vectors(which, name):
    nat = _impl(which)
    cd, sd, post, acc, n_src = FANIN_CASES[name]
    chunks = list(tens(f"{name}_chunks", cd).view(n_src, -1).unbind(0))
    shard = tens(f"{name}_shard", sd)
    if nat is None:
        torch_ops.reduce_scatter_fanin(shard, chunks, post, acc)
    else:
        shard = shard.to("cuda:0")
        nat.post_reduce_fanin(shard, [c.contiguous().to("cuda:0") for c in chunks], post, acc)
    assert_bits_equal(shard, tens(f"{name}_out", sd), name)
