"""Sharded <-> full parameters on one GPU: the logical ranks' flat shards are
reassembled into full parameters by the copy-out kernel, and full parameters
are loaded back fragment by fragment; both directions are byte identities."""

import copy

import pytest
import torch
import torch.nn as nn

from helpers import assert_bits_equal, loc
from test_gpu_fully_shard import DEV, MP, _make

pytestmark = pytest.mark.gpu


def _rank_groups(model0, w, alignment=8):
    from yafsdp_amd import fully_shard

    blocks = []
    for r in range(w):
        blk = copy.deepcopy(model0.blocks[0])
        fully_shard(blk, mesh=(w, r), mp_policy=MP, shard_alignment=alignment)
        blocks.append(blk)
    return blocks, [b._get_fsdp_state()._fsdp_param_group for b in blocks]


@pytest.mark.parametrize("w,alignment", [(1, 8), (3, 8), (5, 1)])
def test_full_tensors_round_trip(w, alignment):
    from yafsdp_amd.checkpoint import full_tensors, group_meta_info, load_full_tensors, sharded_state_dict

    model0 = _make(21)
    want = {n: p.detach().clone() for n, p in model0.blocks[0].named_parameters()}
    blocks, groups = _rank_groups(model0, w, alignment)
    full = full_tensors(groups)
    assert set(full) == set(want)
    for k in want:
        assert_bits_equal(full[k], want[k], f"full tensor {k}")
    # chunks of the ranks' sharded state dicts tile each flattened parameter
    for k in want:
        pieces = []
        for g in groups:
            local, meta = sharded_state_dict(g)[k]
            assert local.numel() == meta.sizes[0] and meta.size == (want[k].numel(),)
            if meta.sizes[0]:
                assert_bits_equal(local, want[k].view(-1)[meta.offsets[0] : meta.offsets[0] + meta.sizes[0]], k)
                pieces.append(local)
        assert_bits_equal(torch.cat(pieces), want[k].view(-1), f"chunks of {k}")
    info = group_meta_info(groups[w - 1])
    assert info["numels"] == [p.numel() for p in want.values()] and info["fqns"] == list(want)
    assert info["shard_boundaries"][1] == info["padded_numel"]
    # load new values into every rank and read them back
    gen = torch.Generator(device=DEV).manual_seed(22)
    new = {k: torch.randn(v.shape, device=DEV, generator=gen) for k, v in want.items()}
    load_full_tensors(groups, new)
    out = {k: torch.empty_like(v) for k, v in new.items()}
    again = full_tensors(groups, out=out)
    for k in new:
        assert again[k] is out[k]
        assert_bits_equal(again[k], new[k], f"reloaded {k}")
    # pad lanes of the last rank's shard stay zero
    lay = groups[0].layout
    pad = lay.pad_numel(w - 1)
    if pad:
        assert float(groups[w - 1]._padded_sharded_param_data[None][-pad:].abs().max()) == 0.0


def test_load_casts_to_the_master_dtype_and_resets_the_copy_in_flag():
    from yafsdp_amd import fully_shard
    from yafsdp_amd.checkpoint import fsdp_groups_of, load_full_tensors

    model = _make(23)
    for b in model.blocks:
        fully_shard(b, mp_policy=MP)
    fully_shard(model.norm, mp_policy=MP)
    fully_shard(model, mp_policy=MP)
    x = torch.randn(4, 128, device=DEV)
    model(x)
    groups = fsdp_groups_of(model)
    g = groups[0]
    for m in (model.blocks[2], model.norm):
        m.reshard()
    full16 = {p._param_fqn: torch.randn(p._orig_size, device=DEV).bfloat16() for p in g.fsdp_params}
    load_full_tensors(g, full16)
    for p in g.fsdp_params:
        assert_bits_equal(p._sharded_param_data, full16[p._param_fqn].float().view(-1), p._param_fqn)
    model(x)  # the forward casts the new masters into the all-gather input
    torch.cuda.synchronize()
    assert_bits_equal(g._all_gather_input[None], g._padded_sharded_param_data[None].bfloat16(), "copy-in after load")
    with pytest.raises(KeyError):
        load_full_tensors(g, {})


def test_full_state_dict_round_trip_through_the_unwrapped_model():
    """Train a wrapped model, save a plain state dict, load it into (a) the unwrapped torch model and (b) a
    freshly wrapped one: all three give the same outputs / masters."""
    from yafsdp_amd import fully_shard
    from yafsdp_amd.checkpoint import full_state_dict, load_full_state_dict

    def wrap(m):
        for b in m.blocks:
            fully_shard(b, mp_policy=MP)
        fully_shard(m.norm, mp_policy=MP)
        return fully_shard(m, mp_policy=MP)

    model0 = _make(24)
    model = wrap(copy.deepcopy(model0))
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    x = torch.randn(8, 128, device=DEV)
    for _ in range(2):
        model(x).float().pow(2).mean().backward()
        opt.step()
        opt.zero_grad(set_to_none=True)
    sd = full_state_dict(model)
    plain = copy.deepcopy(model0)
    plain.load_state_dict(sd)  # names and shapes are those of the unwrapped model
    for k, v in plain.state_dict().items():
        assert_bits_equal(v, sd[k], k)
    fresh = wrap(copy.deepcopy(model0))
    load_full_state_dict(fresh, sd)
    y1, y2 = model(x), fresh(x)
    assert_bits_equal(y2, y1.detach(), "outputs after reload")
    for m in (fresh.blocks[2], fresh.norm):
        m.reshard()  # a forward without a backward leaves the last users of the buffers unsharded
    with pytest.raises(KeyError):
        load_full_state_dict(fresh, {})
    fresh.blocks[1].unshard()
    with pytest.raises(RuntimeError, match="sharded state"):
        full_state_dict(fresh)


def test_dcp_through_module_state_dict_and_the_sharded_parameter_surface(tmp_path):
    """model.state_dict() of a fully_shard model holds the sharded parameters themselves: torch.distributed.checkpoint
    saves and loads them without any helper; p.to_local(), p.placements and p.full_tensor() are the reference's."""
    import torch.distributed.checkpoint as dcp

    from yafsdp_amd import RaggedShardDTensor, fully_shard
    from yafsdp_amd.checkpoint import RaggedShardLoadPlanner, fsdp_groups_of

    def wrap(m):
        for b in m.blocks:
            fully_shard(b, mp_policy=MP)
        fully_shard(m.norm, mp_policy=MP)
        return fully_shard(m, mp_policy=MP)

    model0 = _make(33)
    model = wrap(copy.deepcopy(model0))
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    x = torch.randn(8, 128, device=DEV)
    for _ in range(2):
        model(x).float().pow(2).mean().backward()
        opt.step()
        opt.zero_grad(set_to_none=True)
    for (name, p), (_, p0) in zip(model.named_parameters(), model0.named_parameters()):
        assert isinstance(p, RaggedShardDTensor) and p.shape == p0.shape
        (placement,) = p.placements
        assert (placement.local_numel, placement.global_offset, placement.shard_numels) == (p0.numel(), 0, (p0.numel(),))
        with pytest.raises(NotImplementedError):
            p.to_local()  # under autograd, as in the reference (ya_fsdp/_tensor.py:318-321)
        with torch.no_grad():
            local = p.to_local()
        assert local.dim() == 1 and local.numel() == p0.numel()
        full = p.full_tensor()
        assert full.shape == p0.shape and full.data_ptr() != local.data_ptr()
        assert_bits_equal(full.reshape(-1), local, name)
    sd = model.state_dict()
    assert all(isinstance(v, RaggedShardDTensor) for k, v in sd.items())
    dcp.save(sd, checkpoint_id=str(tmp_path / "ckpt"), no_dist=True)
    fresh = wrap(copy.deepcopy(model0))
    fresh(x)
    for m in (fresh.blocks[2], fresh.norm):
        m.reshard()
    dcp.load(fresh.state_dict(), checkpoint_id=str(tmp_path / "ckpt"), no_dist=True, planner=RaggedShardLoadPlanner())
    for g in fsdp_groups_of(fresh):
        g._all_gather_input_set_dtypes.clear()
    for ga, gb in zip(fsdp_groups_of(model), fsdp_groups_of(fresh)):
        assert_bits_equal(gb._padded_sharded_param_data[None], ga._padded_sharded_param_data[None], "masters")
    assert_bits_equal(fresh(x), model(x).detach(), "outputs after reload")
    # an ordinary state dict of full tensors loads as well: every rank keeps its fragment
    for m in (fresh.blocks[2], fresh.norm, model.blocks[2], model.norm):
        m.reshard()
    fresh.load_state_dict(model0.state_dict())
    for g, (_, p0) in zip([fp for gr in fsdp_groups_of(fresh) for fp in gr.fsdp_params], model0.named_parameters()):
        assert_bits_equal(g._sharded_param_data, p0.detach().reshape(-1), "loaded from full tensors")


def test_full_state_dict_leaves_non_persistent_buffers_out():
    """Buffers registered with persistent=False (rotary tables and the like) are not part of module.state_dict();
    the full state dict follows it, so an ordinary state dict loads with strict=True."""
    from yafsdp_amd import fully_shard
    from yafsdp_amd.checkpoint import full_state_dict, load_full_state_dict

    class WithBuffers(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.Linear(64, 64)
            self.register_buffer("scale", torch.full((64,), 2.0))
            self.register_buffer("inv_freq", torch.arange(64.0), persistent=False)

        def forward(self, x):
            return self.lin(x) * self.scale + self.inv_freq

    torch.manual_seed(31)
    plain = WithBuffers().to(DEV)
    model = fully_shard(copy.deepcopy(plain), mp_policy=MP)
    sd = full_state_dict(model)
    assert sorted(sd) == sorted(plain.state_dict()) and "inv_freq" not in sd
    fresh = fully_shard(WithBuffers().to(DEV), mp_policy=MP)
    load_full_state_dict(fresh, plain.state_dict(), strict=True)
    x = torch.randn(4, 64, device=DEV)
    assert_bits_equal(fresh(x), model(x).detach(), "outputs after loading an ordinary state dict")


def test_torch_distributed_checkpoint_round_trip(tmp_path):
    """A trained wrapped model saved with torch.distributed.checkpoint through its own sharded parameters
    (RaggedShardDTensor: local fragments that are views of the flat master shards, and the checkpoint hooks of
    ya_fsdp/_tensor.py:365-432) and loaded into a freshly wrapped model and into plain flattened tensors."""
    import torch.distributed.checkpoint as dcp

    from yafsdp_amd import fully_shard
    from yafsdp_amd.checkpoint import RaggedShardLoadPlanner, checkpointable_state_dict, fsdp_groups_of

    def wrap(m):
        for b in m.blocks:
            fully_shard(b, mp_policy=MP)
        fully_shard(m.norm, mp_policy=MP)
        return fully_shard(m, mp_policy=MP)

    def handles(m):
        out = {}
        for g in fsdp_groups_of(m):
            out.update(checkpointable_state_dict(g))
        return out

    model0 = _make(31)
    model = wrap(copy.deepcopy(model0))
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    x = torch.randn(8, 128, device=DEV)
    for _ in range(2):
        model(x).float().pow(2).mean().backward()
        opt.step()
        opt.zero_grad(set_to_none=True)
    sd = handles(model)
    assert set(sd) == {n for n, _ in model0.named_parameters()}
    assert all(h.size() == p.size() and loc(h).numel() == p.numel() for h, p in ((sd[n], p) for n, p in model0.named_parameters()))
    with pytest.raises(NotImplementedError, match="dispatch"):
        sd["norm.weight"].sin()
    dcp.save(sd, checkpoint_id=str(tmp_path / "ckpt"), no_dist=True)
    # (a) plain flattened tensors
    flat = {n: torch.full((p.numel(),), float("nan"), device=DEV) for n, p in model0.named_parameters()}
    dcp.load(flat, checkpoint_id=str(tmp_path / "ckpt"), no_dist=True)
    for n, h in sd.items():
        assert_bits_equal(flat[n], loc(h), n)
    # (b) a freshly wrapped model: the load writes its flat master shards
    fresh = wrap(copy.deepcopy(model0))
    fresh(x)  # lazy init (then hand the buffers back, as after any forward without backward)
    for m in (fresh.blocks[2], fresh.norm):
        m.reshard()
    from torch.distributed.checkpoint.api import CheckpointException

    with pytest.raises(CheckpointException, match="Size mismatch"):  # the default planner wants the flattened size
        dcp.load(handles(fresh), checkpoint_id=str(tmp_path / "ckpt"), no_dist=True)
    dcp.load(handles(fresh), checkpoint_id=str(tmp_path / "ckpt"), no_dist=True, planner=RaggedShardLoadPlanner())
    for g in fsdp_groups_of(fresh):
        g._all_gather_input_set_dtypes.clear()
    for ga, gb in zip(fsdp_groups_of(model), fsdp_groups_of(fresh)):
        assert_bits_equal(gb._padded_sharded_param_data[None], ga._padded_sharded_param_data[None], "masters")
    assert_bits_equal(fresh(x), model(x).detach(), "outputs after reload")
