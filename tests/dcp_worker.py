"""One rank of a ``torch.distributed.checkpoint`` save (CPU tensors, gloo): the rank's ragged fragments of a
seeded set of parameters, wrapped as ``RaggedShardTensor``.  Launched by tests/test_checkpoint_dcp.py:

    python dcp_worker.py <checkpoint dir> <world size> <rank> <alignment> <port> <numel> [<numel> ...]
"""

import sys

import torch
import torch.distributed as dist
import torch.distributed.checkpoint as dcp


def full_parameters(numels, seed=4242):
    g = torch.Generator().manual_seed(seed)
    return {f"layer.p{i}": torch.randn(n, generator=g) for i, n in enumerate(numels)}


def rank_state_dict(numels, world_size, rank, alignment, fill=None):
    """This rank's fragments (slices of the flat padded buffer), as checkpointable tensors."""
    from yafsdp_amd._layout import make_layout
    from yafsdp_amd.checkpoint import RaggedShardTensor, chunk_meta

    lay = make_layout(numels, world_size, alignment)
    full = full_parameters(numels)
    flat = torch.zeros(lay.padded_unsharded_numel)
    flat[: lay.total_numel] = torch.cat([full[f"layer.p{i}"] for i in range(len(numels))])
    lo, _ = lay.rank_range(rank)
    shard = flat[lo : lo + lay.padded_sharded_numel].clone()
    if fill is not None:
        shard.fill_(fill)
    out, pos = {}, 0
    for i, (n, placement) in enumerate(zip(lay.sharded_numels(rank), lay.placements(rank))):
        meta = chunk_meta(f"layer.p{i}", placement, (numels[i],))
        out[meta.fqn] = RaggedShardTensor.wrap(shard[pos : pos + n], meta)
        pos += n
    return out, shard


def main():
    path, world_size, rank, alignment, port = sys.argv[1], int(sys.argv[2]), int(sys.argv[3]), int(sys.argv[4]), sys.argv[5]
    numels = [int(a) for a in sys.argv[6:]]
    dist.init_process_group("gloo", init_method=f"tcp://127.0.0.1:{port}", rank=rank, world_size=world_size)
    try:
        state_dict, _ = rank_state_dict(numels, world_size, rank, alignment)
        dcp.save(state_dict, checkpoint_id=path)
    finally:
        dist.destroy_process_group()
    print("saved", rank, flush=True)


if __name__ == "__main__":
    main()
