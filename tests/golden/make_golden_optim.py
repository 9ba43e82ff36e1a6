"""Writes ``tests/golden/optim_small.npz``: small inputs and expected outputs of
the optimizer-side passes and of the reduce fan-in.

Expected values of the Adam(W) step, the sum of squares, the clip coefficient
and the scaling come from the plain-C restatement (``oracle.cref``); the Adam
vectors are accepted only if the torch-op sequence of ``torch.optim`` on CPU
gives bit-identical moments and parameters within two ulps of the update
(torch's CPU square root is not correctly rounded).  The fan-in vectors come
from the torch-op oracle.  Nothing here was produced by running the reference.
Arrays are raw bit patterns (uint16 / uint32) or float64 / float32 scalars,
loadable with ``numpy.load(allow_pickle=False)``.

Run from the repository root:  python tests/golden/make_golden_optim.py
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import cref, torch_ops  # noqa: E402
from tests.helpers import assert_bits_equal, mixed_values  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "optim_small.npz")
NAMES = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}

ADAM_CASES = {
    # name: (decoupled, beta1, weight_decay, step, out16 dtype or None, grad_scale or None, zero_grad)
    "adamw_first": (True, 0.9, 0.1, 1, torch.bfloat16, None, False),
    "adamw_scaled": (True, 0.9, 0.1, 7, torch.float16, 0.37, True),
    "adam_l2": (False, 0.3, 0.01, 3, None, None, False),
}
HP = dict(lr=3e-4, beta2=0.95, eps=1e-8)


def bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.float32:
        return t.contiguous().view(torch.int32).numpy().view(np.uint32).copy()
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def main() -> None:
    g = torch.Generator().manual_seed(4343)
    data = {}
    n = 300
    for name, (decoupled, beta1, wd, step, out_dt, gscale, zero) in ADAM_CASES.items():
        p = torch.randn(n, generator=g) * 0.02
        grad = torch.randn(n, generator=g) * 1e-3
        m = torch.randn(n, generator=g) * 1e-3
        v = (torch.randn(n, generator=g) * 1e-3) ** 2
        p[:4] = torch.tensor([0.0, -0.0, 1e-40, 3.0])
        grad[:4] = torch.tensor([0.0, 1e-42, -2.0, 0.0])
        for key, t in (("p", p), ("g", grad), ("m", m), ("v", v)):
            data[f"{name}_{key}_in"] = bits(t)
        op, og, om, ov = p.clone(), grad.clone(), m.clone(), v.clone()
        out16 = None if out_dt is None else torch.zeros(n, dtype=out_dt)
        cref.adamw_step(op, og, om, ov, out16, lr=HP["lr"], beta1=beta1, beta2=HP["beta2"], eps=HP["eps"],
                        weight_decay=wd, step=step, decoupled=decoupled, grad_scale=gscale, zero_grad=zero)
        # cross-check against torch's own op sequence
        tp, tm, tv = p.clone(), m.clone(), v.clone()
        tg = grad.clone() if gscale is None else grad.clone().mul_(torch.tensor(gscale))
        torch_ops.adam_step_torch_ops(tp, tg, tm, tv, lr=HP["lr"], beta1=beta1, beta2=HP["beta2"], eps=HP["eps"],
                                      weight_decay=wd, step=step, decoupled=decoupled)
        assert_bits_equal(om, tm, name + " exp_avg"), assert_bits_equal(ov, tv, name + " exp_avg_sq")
        scale = torch.maximum(tp.abs(), (tp - p).abs()).double()
        assert bool(((op.double() - tp.double()).abs() <= 2.0**-22 * scale).all()), name
        for key, t in (("p", op), ("g", og), ("m", om), ("v", ov)):
            data[f"{name}_{key}_out"] = bits(t)
        if out16 is not None:
            data[f"{name}_out16"] = bits(out16)
    for dt in NAMES:
        x = mixed_values(g, n, dt, 3e-2)[40:].contiguous()  # finite values only
        x[x.float().abs() > 1e3] = 1.0
        data[f"sumsq_{NAMES[dt]}_in"] = bits(x)
        data[f"sumsq_{NAMES[dt]}_out"] = np.array([cref.sumsq(x)], dtype=np.float64)
        y = x.clone()
        cref.flat_scale(y, 0.7334219)
        want = x.clone().mul_(torch.tensor(0.7334219))
        assert_bits_equal(y, want, "scale")
        data[f"scale_{NAMES[dt]}_out"] = bits(y)
    for k, (sumsq, max_norm) in enumerate([(27.259829024930415, 1.0), (1e-8, 1.0), (4.0, 0.5)]):
        norm, coef = cref.clip_coef(sumsq, max_norm)
        data[f"clip_{k}"] = np.array([sumsq, max_norm], dtype=np.float64)
        data[f"clip_{k}_out"] = np.array([norm, coef], dtype=np.float32)
    for name, (cd, sd, post, acc, n_src) in {"fanin_bf16": (torch.bfloat16, torch.float32, 8.0, True, 8),
                                             "fanin_f32": (torch.float32, torch.bfloat16, 3.0, False, 3)}.items():
        chunks = [mixed_values(g, n, cd, 1e-3).roll(k) for k in range(n_src)]
        shard = mixed_values(g, n, sd, 1e-4).flip(0).contiguous()
        want = shard.clone()
        torch_ops.reduce_scatter_fanin(want, chunks, post, acc)
        data[f"{name}_chunks"] = bits(torch.stack(chunks).reshape(-1))
        data[f"{name}_shard"], data[f"{name}_out"] = bits(shard), bits(want)
    np.savez_compressed(OUT, **data)
    print(OUT, os.path.getsize(OUT), "bytes,", len(data), "arrays")


if __name__ == "__main__":
    main()
