"""Brute-force ragged split for tiny inputs: TEST INFRASTRUCTURE ONLY.

Restates the *method* of ya_fsdp/_param_group.py:284-377 with numpy: one
parameter index and one element index per element of the padded buffer, the
buffer chunked evenly over the ranks, counts by equality and offsets by minimum.
It shares no arithmetic with the closed form in ``yafsdp_amd/_layout.py``.
"""

from __future__ import annotations

import numpy as np

_NO_PARAM = np.iinfo(np.uint16).max
_NO_ELEM = np.iinfo(np.int64).max


def bruteforce_layout(numels, world_size: int, shard_alignment: int, rank: int):
    numels = [int(n) for n in numels]
    total = sum(numels)
    divider = world_size * shard_alignment  # :251
    padded = total
    if padded % divider != 0:  # :252-255
        padded += divider - padded % divider
    shard = padded // world_size  # :259-261

    param_idx = np.full(padded, _NO_PARAM, dtype=np.uint16)  # :290-294
    elem_idx = np.full(padded, _NO_ELEM, dtype=np.int64)  # :295-299
    pos = 0
    for p, n in enumerate(numels):  # :300-332
        param_idx[pos : pos + n] = p
        elem_idx[pos : pos + n] = np.arange(n, dtype=np.int64)
        pos += n

    per_rank_param_idx = np.split(param_idx, world_size)  # torch.chunk on a divisible length, :340-342
    per_rank_elem_idx = np.split(elem_idx, world_size)
    mine_p, mine_e = per_rank_param_idx[rank], per_rank_elem_idx[rank]

    per_rank_sharded_numels = [  # :347-353
        tuple(int((chunk == p).sum()) for chunk in per_rank_param_idx) for p in range(len(numels))
    ]
    sharded_numels = [int((mine_p == p).sum()) for p in range(len(numels))]  # :354-358
    global_offsets = []
    for p in range(len(numels)):  # :359-377
        sel = mine_e[mine_p == p]
        global_offsets.append(int(sel.min()) if sel.size > 0 else numels[p])
    return {
        "total": total,
        "padded": padded,
        "shard": shard,
        "sharded_numels": sharded_numels,
        "global_offsets": global_offsets,
        "per_rank_sharded_numels": per_rank_sharded_numels,
    }
