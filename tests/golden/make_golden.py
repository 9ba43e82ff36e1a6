"""Writes ``tests/golden/bufpath_small.npz``: small inputs and expected outputs of
every op of the buffer path.

The expected values come from the torch-op oracle (``oracle.torch_ops``) and are
accepted only if the independent plain-C restatement (``oracle.cref``) produces
the same bits.  The reference ships no vectors of its own and cannot be imported
under this interpreter, so nothing here was produced by running it.  Arrays are
stored as raw bit patterns (uint16 / uint32), loadable with
``numpy.load(allow_pickle=False)``.

Run from the repository root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import cref, torch_ops  # noqa: E402
from tests.helpers import assert_bits_equal, mixed_values  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bufpath_small.npz")
NAMES = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}


def bits(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.float32:
        return t.contiguous().view(torch.int32).numpy().view(np.uint32).copy()
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def main() -> None:
    g = torch.Generator().manual_seed(4242)
    data = {}
    n = 200
    # casts: every ordered pair of dtypes
    for sd in NAMES:
        src = mixed_values(g, n, sd, 0.02)
        data[f"cast_src_{NAMES[sd]}"] = bits(src)
        for dd in NAMES:
            want = torch.empty(n, dtype=dd)
            torch_ops.copy_in(want, src)
            chk = torch.empty(n, dtype=dd)
            cref.flat_copy(chk, src)
            assert_bits_equal(want, chk, f"cast {sd}->{dd}")
            data[f"cast_{NAMES[sd]}_to_{NAMES[dd]}"] = bits(want)
    # divide and post-reduce
    for dt in NAMES:
        for f in (8.0, 3.0):
            x = mixed_values(g, n, dt, 1e-3)
            y = x.clone()
            torch_ops.div_if_needed(y, f)
            c = x.clone()
            cref.flat_div(c, f)
            assert_bits_equal(y, c, "div")
            data[f"div_{NAMES[dt]}_{int(f)}_in"] = bits(x)
            data[f"div_{NAMES[dt]}_{int(f)}_out"] = bits(y)
    for sd, cd in [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float32, torch.float16)]:
        for post in (0.0, 8.0, 3.0):
            for acc in (0, 1):
                chunk = mixed_values(g, n, cd, 1e-3)
                shard = mixed_values(g, n, sd, 1e-4).flip(0).contiguous()
                want = shard.clone()
                torch_ops.reduce_scatter_local(want, chunk.clone(), 1, 0, None, post or None, "add" if acc else "copy")
                chk = shard.clone()
                cref.post_reduce(chk, chunk, post or None, bool(acc))
                assert_bits_equal(want, chk, "post")
                key = f"post_{NAMES[sd]}_{NAMES[cd]}_{int(post)}_{acc}"
                data[key + "_chunk"], data[key + "_shard"], data[key + "_out"] = bits(chunk), bits(shard), bits(want)
    # gather-in / scatter-out over a ragged table
    numels = [5, 1, 300, 0, 77, 130, 3, 1101]
    t = sum(numels)
    t_pad = t + 13
    offsets = np.concatenate([[0], np.cumsum(numels)])
    modes = [1, 2, 1, 1, 0, 2, 2, 1]
    data["table_numels"] = np.array(numels, dtype=np.int64)
    data["table_modes"] = np.array(modes, dtype=np.uint8)
    data["table_padded"] = np.array([t_pad], dtype=np.int64)
    for gd, rd in [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float32, torch.bfloat16)]:
        for pre in (0.0, 8.0, 3.0):
            grads = [mixed_values(g, k, gd, 1e-3) for k in numels]
            old = torch.zeros(t_pad, dtype=rd)
            old[:t] = mixed_values(g, t, rd, 1e-3).flip(0)
            want = old.clone()
            views = list(want[:t].split(numels))
            cp = [i for i, m in enumerate(modes) if m == 1]
            ad = [i for i, m in enumerate(modes) if m == 2]
            torch_ops.reduce_copy_in([views[i] for i in cp], [grads[i] for i in cp], False)
            torch_ops.reduce_copy_in([views[i] for i in ad], [grads[i] for i in ad], True)
            torch_ops.div_if_needed(want, pre or None)
            chk = old.clone()
            cref.gather_in(grads, modes, offsets, chk, t_pad, pre or None, True)
            assert_bits_equal(want, chk, "gather")
            key = f"gather_{NAMES[gd]}_{NAMES[rd]}_{int(pre)}"
            data[key + "_grads"] = bits(torch.cat(grads))
            data[key + "_old"], data[key + "_out"] = bits(old), bits(want)
    flat = mixed_values(g, t_pad, torch.bfloat16, 0.02)
    outs = [torch.empty(k, dtype=torch.bfloat16) for k in numels]
    torch_ops.copy_out_materialize(flat, numels, outs)
    data["scatter_flat"] = bits(flat)
    data["scatter_out"] = bits(torch.cat(outs))
    np.savez_compressed(OUT, **data)
    print(OUT, os.path.getsize(OUT), "bytes,", len(data), "arrays")


if __name__ == "__main__":
    main()
