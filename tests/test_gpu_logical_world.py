"""Sharded data-parallel training over W logical ranks on ONE GPU.

Every rank is a ``fully_shard``-wrapped replica of the model with ``mesh=(W, r)``: it owns its ragged shard
of every parameter group, runs its own forward and backward on its own micro-batch through the hooks, and
leaves its unreduced gradients in the group's reduce buffer.  The two exchanges that a process group would do
are done here by the test with the one-GPU kernels of those exchange points:

* all-gather: rank r's gathered buffer receives the 16-bit all-gather input of every peer in its slot
  (``flat_copy``, what ``all_gather_into_tensor`` delivers, ya_fsdp/_collectives.py:60-65);
* reduce-scatter: rank r's gradient shard receives ``ReduceOp.AVG`` over all ranks' reduce buffers of chunk r as the
  collective library defines it (a pre-multiplied sum: every rank's element times 1 / W in the reduce dtype, rounded,
  then the sum), added in binary32 in rank order and rounded to the reduce dtype (``post_reduce_fanin(premul=)``:
  ya_fsdp/_collectives.py:152-162 and :243-249 with a binary32 accumulator, then :185).

The masters of all ranks, reassembled, must equal bit for bit those of one unsharded model trained by hand
with the same arithmetic.  No second GPU, no process group, no peer mapping is involved."""

import copy

import pytest
import torch

from helpers import loc
from yafsdp_amd import connect_logical_ranks

from yafsdp_amd import _native, fully_shard
from yafsdp_amd.checkpoint import full_tensors

from test_gpu_fully_shard import DEV, MP, _make

pytestmark = pytest.mark.gpu


def _wrap_rank(model, w, r, alignment):
    kw = dict(mesh=(w, r), mp_policy=MP, shard_alignment=alignment, reshard_after_forward=False)
    for b in model.blocks:
        fully_shard(b, **kw)
    fully_shard(model.norm, **kw)
    return fully_shard(model, **kw)


def _groups(model):
    return [m._get_fsdp_state()._fsdp_param_group for m in (*model.blocks, model.norm)]


def _all_gather(ranks):
    """Every rank unshards every group (copy-in cast + its own slot), then receives its peers' slots."""
    w = len(ranks)
    for model in ranks:
        for m in (*model.blocks, model.norm):
            m.unshard()
    per_rank = [_groups(model) for model in ranks]
    for r in range(w):
        for g, group in enumerate(per_rank[r]):
            s = group.layout.padded_sharded_numel
            out = group._all_gather_output[None]
            for q in range(w):
                if q != r:
                    _native.flat_copy(out[q * s : (q + 1) * s], per_rank[q][g]._all_gather_input[None])


def _reduce_scatter(ranks):
    """Chunk r of every rank's reduce buffer, averaged as the collective does it, into rank r's gradient shard."""
    w = len(ranks)
    per_rank = [_groups(model) for model in ranks]
    for r in range(w):
        for g, group in enumerate(per_rank[r]):
            s = group.layout.padded_sharded_numel
            chunks = [per_rank[q][g]._reduce_scatter_input[None][r * s : (r + 1) * s] for q in range(w)]
            _native.post_reduce_fanin(group._padded_sharded_param_grad[None], chunks, None, False, premul=1.0 / w)
            for fp in group.fsdp_params:
                fp.sharded_param.grad = fp.sharded_param_grad      # ya_fsdp/_collectives.py:216-217
    for groups in per_rank:                                         # the reduce buffers are free again
        for group in groups:
            for fp in group.fsdp_params:
                fp.unsharded_accumulated_grad = None
            group.grad_buffer_ctx.owner = None


def _reference(model0, batches, lr, w):
    """One unsharded model, the same arithmetic by hand: bf16 gradients per micro-batch, each multiplied by
    bf16(1 / W) in bf16, summed over the ranks in binary32 in rank order, rounded to bf16, upcast into the fp32
    gradient, SGD."""
    ref = copy.deepcopy(model0)
    masters = list(ref.parameters())
    opt = torch.optim.SGD(masters, lr=lr)
    scalar = torch.tensor(1.0 / w, dtype=torch.float32).to(torch.bfloat16).to(DEV)
    for xs in batches:
        lowp = copy.deepcopy(ref).to(torch.bfloat16)
        sums = None
        for x in xs:
            for p in lowp.parameters():
                p.grad = None
            lowp(x.to(torch.bfloat16)).float().pow(2).mean().backward()
            grads = [(p.grad * scalar).float() for p in lowp.parameters()]  # bf16 * bf16 -> bf16: one rounding
            sums = grads if sums is None else [a.add_(g) for a, g in zip(sums, grads)]
        for m, a in zip(masters, sums):
            m.grad = a.bfloat16().float()
        opt.step()
        opt.zero_grad(set_to_none=True)
    return ref


@pytest.mark.parametrize("w,alignment", [(2, 8), (3, 8), (4, 1)])
def test_logical_ranks_train_like_one_unsharded_model(w, alignment):
    print("logical world", w, alignment, flush=True)
    model0 = _make(91)
    gen = torch.Generator(device=DEV).manual_seed(500 + w)
    batches = [[torch.randn(8, 128, device=DEV, generator=gen) for _ in range(w)] for _ in range(3)]
    want = dict(_reference(model0, batches, 0.05, w).named_parameters())

    ranks = [_wrap_rank(copy.deepcopy(model0), w, r, alignment) for r in range(w)]
    opts = [torch.optim.SGD(model.parameters(), lr=0.05) for model in ranks]
    for model in ranks:
        model._get_fsdp_state()._lazy_init(allow_no_grad_reduce=True)  # one reduce buffer per group
        model.set_requires_gradient_sync(False)                        # gradients stay unreduced in it
    # every rank's shards together are the model: some parameter is split between ranks
    sizes = [[loc(p).numel() for p in model.parameters()] for model in ranks]
    assert any(0 < a < b for a, b in zip(sizes[0], [p.numel() for p in model0.parameters()]))
    for xs in batches:
        _all_gather(ranks)
        for model, x in zip(ranks, xs):
            model(x).float().pow(2).mean().backward()
        _reduce_scatter(ranks)
        for opt in opts:
            opt.step()
            opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    per_rank = [_groups(model) for model in ranks]
    got = {}
    for g in range(len(per_rank[0])):
        got.update(full_tensors([per_rank[r][g] for r in range(w)]))
    assert set(got) == set(want)
    for k, v in want.items():
        assert torch.equal(got[k].view(torch.int32), v.detach().view(torch.int32)), k
    # the same through the sharded parameters themselves: once the logical ranks know each other, full_tensor() of
    # any rank's parameter assembles the whole parameter from all ranks' fragments (ya_fsdp/_tensor.py:341-363)
    with pytest.raises(RuntimeError, match="connect_logical_ranks"):
        next(p for p in ranks[0].parameters() if 0 < loc(p).numel() < p.numel()).full_tensor()
    connect_logical_ranks(ranks)
    for r in (0, w - 1):
        for k, p in ranks[r].named_parameters():
            assert p.placements[0].shard_numels == tuple(loc(q).numel() for q in
                                                          (dict(m.named_parameters())[k] for m in ranks))
            full = p.full_tensor()
            assert full.shape == want[k].shape and torch.equal(full.view(torch.int32), want[k].detach().view(torch.int32)), k
