"""The sharded checkpoint format against torch's own ``torch.distributed.checkpoint``: two ranks (CPU tensors,
gloo) save their ragged fragments as ``RaggedShardTensor``; the checkpoint is then read back as whole flattened
parameters and as the fragments of other layouts (another world size and alignment).  The chunk each rank
declares is the reference's (ya_fsdp/_tensor.py:365-432); torch's planner validates that the chunks of all
ranks tile every parameter exactly, and its resharding reads prove the offsets."""

import os
import socket
import subprocess
import sys

import pytest
import torch
import torch.distributed.checkpoint as dcp

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from dcp_worker import full_parameters, rank_state_dict  # noqa: E402

NUMELS = [37, 5, 1, 260, 64, 3]  # W = 2, alignment 8: the boundary falls inside p3; p0..p2 live on rank 0 only


def _free_port():
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


@pytest.fixture(scope="module")
def checkpoint(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("dcp") / "ckpt")
    port = str(_free_port())
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([os.path.dirname(HERE), os.environ.get("PYTHONPATH", "")]))
    procs = [
        subprocess.Popen([sys.executable, os.path.join(HERE, "dcp_worker.py"), path, "2", str(r), "8", port,
                          *map(str, NUMELS)], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        for r in range(2)
    ]
    outs = []
    for p in procs:
        try:
            out, _ = p.communicate(timeout=180)
        except subprocess.TimeoutExpired:
            for q in procs:
                q.kill()
            raise
        outs.append(out)
    assert all(p.returncode == 0 for p in procs), "\n".join(outs)
    return path


def test_saved_metadata_holds_the_chunks_of_both_ranks(checkpoint):
    from torch.distributed.checkpoint import FileSystemReader

    md = FileSystemReader(checkpoint).read_metadata()
    from yafsdp_amd._layout import make_layout
    from yafsdp_amd.checkpoint import chunk_meta

    lay = make_layout(NUMELS, 2, 8)
    for i, n in enumerate(NUMELS):
        entry = md.state_dict_metadata[f"layer.p{i}"]
        assert tuple(entry.size) == (n,)
        got = sorted((tuple(c.offsets), tuple(c.sizes)) for c in entry.chunks)
        want = sorted(
            (m.offsets, m.sizes) for m in (chunk_meta("x", lay.placements(r)[i], (n,)) for r in range(2))
        )
        assert got == want, (i, got, want)


def test_whole_parameters_come_back(checkpoint):
    want = full_parameters(NUMELS)
    got = {k: torch.full_like(v, float("nan")) for k, v in want.items()}
    dcp.load(got, checkpoint_id=checkpoint, no_dist=True)
    for k in want:
        assert torch.equal(got[k], want[k]), k


@pytest.mark.parametrize("world_size,alignment", [(3, 1), (5, 2), (1, 8)])
def test_fragments_of_another_layout_come_back(checkpoint, world_size, alignment):
    """Resharding: every rank of a different layout reads exactly its own fragments."""
    for rank in range(world_size):
        want, want_shard = rank_state_dict(NUMELS, world_size, rank, alignment)
        got, got_shard = rank_state_dict(NUMELS, world_size, rank, alignment, fill=float("nan"))
        dcp.load(got, checkpoint_id=checkpoint, no_dist=True)
        real = sum(v.local_tensor.numel() for v in want.values())  # the pad lanes behind the fragments are not part of any chunk
        assert torch.equal(got_shard[:real], want_shard[:real]), (world_size, rank)
        assert torch.isnan(got_shard[real:]).all()
