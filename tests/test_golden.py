"""Committed golden vectors (tests/golden/bufpath_small.npz, written by
tests/golden/make_golden.py from the torch-op oracle and cross-checked against
the plain-C restatement at generation time).

CPU: the oracle and the C restatement still reproduce them (guards against a
torch upgrade changing an op).  GPU: the HIP path reproduces them through the C
ABI."""

import os

import numpy as np
import pytest
import torch

from oracle import cref, torch_ops
from tests.helpers import assert_bits_equal

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "bufpath_small.npz"),
               allow_pickle=False)
DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
PAIRS_POST = [("f32", "bf16"), ("bf16", "f32"), ("f32", "f16")]
PAIRS_GATHER = [("bf16", "bf16"), ("bf16", "f32"), ("f32", "bf16")]


def tens(key: str, name: str) -> torch.Tensor:
    a = GOLD[key]
    if name == "f32":
        return torch.from_numpy(a.view(np.int32).copy()).view(torch.float32)
    return torch.from_numpy(a.view(np.int16).copy()).view(DT[name])


class CpuImpl:
    """oracle.torch_ops and oracle.cref, each must match the vectors."""

    def __init__(self, use_c):
        self.use_c = use_c
        self.dev = "cpu"

    def cast(self, dst, src):
        cref.flat_copy(dst, src) if self.use_c else torch_ops.copy_in(dst, src)

    def div(self, buf, f):
        cref.flat_div(buf, f) if self.use_c else torch_ops.div_if_needed(buf, f)

    def post(self, shard, chunk, post, acc):
        if self.use_c:
            cref.post_reduce(shard, chunk, post, acc)
        else:
            torch_ops.reduce_scatter_local(shard, chunk.clone(), 1, 0, None, post, "add" if acc else "copy")

    def gather(self, numels, padded, grads, modes, flat, pre):
        t = sum(numels)
        if self.use_c:
            cref.gather_in(grads, modes, np.concatenate([[0], np.cumsum(numels)]), flat, padded, pre, True)
            return
        views = list(flat[:t].split(numels))
        cp = [i for i, m in enumerate(modes) if m == 1]
        ad = [i for i, m in enumerate(modes) if m == 2]
        torch_ops.reduce_copy_in([views[i] for i in cp], [grads[i] for i in cp], False)
        torch_ops.reduce_copy_in([views[i] for i in ad], [grads[i] for i in ad], True)
        torch_ops.div_if_needed(flat, pre)

    def scatter(self, numels, padded, flat, outs):
        if self.use_c:
            cref.scatter_out(outs, np.concatenate([[0], np.cumsum(numels)]), flat)
        else:
            torch_ops.copy_out_materialize(flat, numels, outs)


class HipImpl:
    def __init__(self):
        from yafsdp_amd import _native

        self.n = _native
        self.dev = "cuda:0"

    def cast(self, dst, src):
        self.n.flat_copy(dst, src)

    def div(self, buf, f):
        self.n.flat_div(buf, f)

    def post(self, shard, chunk, post, acc):
        self.n.post_reduce(shard, chunk, post, acc)

    def gather(self, numels, padded, grads, modes, flat, pre):
        self.n.TensorTable(numels, padded, torch.device(self.dev)).gather_in(grads, flat, modes, pre, True)

    def scatter(self, numels, padded, flat, outs):
        self.n.TensorTable(numels, padded, torch.device(self.dev)).scatter_out(flat, outs)


def run_all(impl):
    dev = impl.dev
    for s in DT:
        src = tens(f"cast_src_{s}", s).to(dev)
        for d in DT:
            out = torch.empty(src.numel(), dtype=DT[d], device=dev)
            impl.cast(out, src)
            assert_bits_equal(out, tens(f"cast_{s}_to_{d}", d), f"cast {s}->{d}")
    for d in DT:
        for f in (8, 3):
            buf = tens(f"div_{d}_{f}_in", d).to(dev)
            impl.div(buf, float(f))
            assert_bits_equal(buf, tens(f"div_{d}_{f}_out", d), f"div {d} /{f}")
    for sd, cd in PAIRS_POST:
        for post in (0, 8, 3):
            for acc in (0, 1):
                key = f"post_{sd}_{cd}_{post}_{acc}"
                shard = tens(key + "_shard", sd).to(dev)
                impl.post(shard, tens(key + "_chunk", cd).to(dev), float(post) or None, bool(acc))
                assert_bits_equal(shard, tens(key + "_out", sd), key)
    numels = GOLD["table_numels"].tolist()
    modes = GOLD["table_modes"].tolist()
    padded = int(GOLD["table_padded"][0])
    for gd, rd in PAIRS_GATHER:
        for pre in (0, 8, 3):
            key = f"gather_{gd}_{rd}_{pre}"
            grads = [g.contiguous().to(dev) for g in tens(key + "_grads", gd).split(numels)]
            flat = tens(key + "_old", rd).to(dev)
            impl.gather(numels, padded, grads, modes, flat, float(pre) or None)
            assert_bits_equal(flat, tens(key + "_out", rd), key)
    flat = tens("scatter_flat", "bf16").to(dev)
    outs = [torch.empty(n, dtype=torch.bfloat16, device=dev) for n in numels]
    impl.scatter(numels, padded, flat, outs)
    assert_bits_equal(torch.cat(outs), tens("scatter_out", "bf16"), "scatter")


@pytest.mark.parametrize("use_c", [False, True], ids=["torch-ops", "plain-c"])
def test_oracle_reproduces_golden(use_c):
    run_all(CpuImpl(use_c))


@pytest.mark.gpu
def test_hip_reproduces_golden():
    run_all(HipImpl())
