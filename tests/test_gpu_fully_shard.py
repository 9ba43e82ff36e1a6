"""``fully_shard`` on one GPU: a wrapped model trains through the buffer
kernels and its master weights stay bit-identical to a hand-written mixed
precision loop that performs the same arithmetic with plain torch ops."""

import copy

import pytest
import torch
import torch.nn as nn

from helpers import loc
from yafsdp_amd import MixedPrecisionPolicy, make_layout
from yafsdp_amd._tensor import RaggedShardDTensor

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


class Block(nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.up = nn.Linear(d, h)
        self.down = nn.Linear(h, d, bias=False)

    def forward(self, x):
        return x + self.down(torch.relu(self.up(x)))


class Net(nn.Module):
    def __init__(self, d=128, h=256, layers=3):
        super().__init__()
        self.blocks = nn.ModuleList([Block(d, h) for _ in range(layers)])
        self.norm = nn.LayerNorm(d)

    def forward(self, x):
        for b in self.blocks:
            x = b(x)
        return self.norm(x)


def _make(seed=0):
    torch.manual_seed(seed)
    return Net().to(DEV)


def _wrap(model, **kw):
    from yafsdp_amd import fully_shard

    for b in model.blocks:
        fully_shard(b, **kw)
    fully_shard(model.norm, **kw)
    return fully_shard(model, **kw)  # the root holds no parameters of its own: siblings only


def _reference_steps(model0, xs, lr, accumulate_pairs=False, reduce_fp32=False):
    """fp32 masters; bf16 compute copies; bf16 gradients (summed over the micro-batches of a step in the dtype of
    the reduce buffer: bf16, or fp32 with ``reduce_dtype=torch.float32``) upcast into fp32; SGD on the masters."""
    ref = copy.deepcopy(model0)
    masters = [p for p in ref.parameters()]
    opt = torch.optim.SGD(masters, lr=lr)
    micro = 2 if accumulate_pairs else 1
    for i in range(0, len(xs), micro):
        acc = None
        for x in xs[i : i + micro]:
            lowp = copy.deepcopy(ref).to(torch.bfloat16)
            y = lowp(x.to(torch.bfloat16))
            y.float().pow(2).mean().backward()
            grads = [None if p.grad is None else (p.grad.float() if reduce_fp32 else p.grad) for p in lowp.parameters()]
            if acc is None:
                acc = [None if g is None else g.clone() for g in grads]   # view.copy_(grad)
            else:
                for a, g in zip(acc, grads):
                    if g is not None:
                        a.add_(g)                         # view.add_(grad): bf16 result
        for m, a in zip(masters, acc):
            m.grad = None if a is None else a.float()     # shard.copy_(chunk): exact upcast
        opt.step()
        opt.zero_grad(set_to_none=True)
    return ref


def _gather_full(model):
    """Full fp32 master values per original parameter name, read back from the flat shards (W=1)."""
    from yafsdp_amd.fully_shard import YaFSDPModule

    out = {}
    for mod in model.modules():
        if isinstance(mod, YaFSDPModule) and (group := mod._get_fsdp_state()._fsdp_param_group) is not None:
            for fp in group.fsdp_params:
                out[fp._param_fqn] = fp._sharded_param_data.detach().view(fp._orig_size).clone()
    return out


MP = MixedPrecisionPolicy(param_dtype=torch.bfloat16, cast_forward_inputs=True)


def test_training_is_bit_identical_to_manual_mixed_precision():
    model0 = _make()
    xs = [torch.randn(16, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(s)) for s in range(4)]
    ref = _reference_steps(model0, xs, lr=0.05)
    model = _wrap(copy.deepcopy(model0), mp_policy=MP)
    # the optimizer sees one fp32 sharded parameter per original parameter: it stands for the whole parameter (its
    # shape) and holds this rank's 1-D fragment of the flat master shard
    params = list(model.parameters())
    assert all(isinstance(p, RaggedShardDTensor) and p.dtype == torch.float32 and loc(p).dim() == 1 for p in params)
    assert [p.shape for p in params] == [p.shape for p in model0.parameters()]
    assert sum(loc(p).numel() for p in params) == sum(p.numel() for p in model0.parameters())
    opt = torch.optim.SGD(params, lr=0.05)
    for x in xs:
        y = model(x)
        assert y.dtype == torch.bfloat16
        y.float().pow(2).mean().backward()
        assert all(p.grad is not None and p.grad.dtype == torch.float32 for p in params)
        opt.step()
        opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    got = _gather_full(model)
    want = dict(ref.named_parameters())
    assert set(got) == set(want)
    for k in want:
        assert torch.equal(got[k].view(torch.int32), want[k].detach().view(torch.int32)), k


def test_gradient_accumulation_without_sync():
    model0 = _make(1)
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(10 + s)) for s in range(4)]
    ref = _reference_steps(model0, xs, lr=0.02, accumulate_pairs=True)
    model = _wrap(copy.deepcopy(model0), mp_policy=MP)
    params = list(model.parameters())
    opt = torch.optim.SGD(params, lr=0.02)
    # unreduced gradients stay in the reduce buffer between micro-batches: one buffer per group
    model._get_fsdp_state()._lazy_init(allow_no_grad_reduce=True)
    for i in range(0, 4, 2):
        model.set_requires_gradient_sync(False)
        model.set_is_last_backward(False)
        model(xs[i]).float().pow(2).mean().backward()          # accumulate in the unsharded reduce buffers... 
        model.set_requires_gradient_sync(True)
        model.set_is_last_backward(True)
        model(xs[i + 1]).float().pow(2).mean().backward()      # ...then reduce once
        opt.step()
        opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    got, want = _gather_full(model), dict(ref.named_parameters())
    assert set(got) == set(want)
    for k in want:
        assert torch.equal(got[k].view(torch.int32), want[k].detach().view(torch.int32)), k


def test_fp32_reduce_buffer_with_accumulation():
    """param_dtype=bf16, reduce_dtype=fp32: gradients are upcast on their way into the reduce buffer and the
    micro-batches of a step add up in fp32 there."""
    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.float32, cast_forward_inputs=True)
    model0 = _make(6)
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(70 + s)) for s in range(4)]
    ref = _reference_steps(model0, xs, lr=0.02, accumulate_pairs=True, reduce_fp32=True)
    model = _wrap(copy.deepcopy(model0), mp_policy=mp)
    opt = torch.optim.SGD(model.parameters(), lr=0.02)
    model._get_fsdp_state()._lazy_init(allow_no_grad_reduce=True)
    for i in range(0, 4, 2):
        model.set_requires_gradient_sync(False)
        model.set_is_last_backward(False)
        model(xs[i]).float().pow(2).mean().backward()
        model.set_requires_gradient_sync(True)
        model.set_is_last_backward(True)
        model(xs[i + 1]).float().pow(2).mean().backward()
        opt.step()
        opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    group = model.blocks[0]._get_fsdp_state()._fsdp_param_group
    assert group.reduce_scatter_dtype == torch.float32 and group.all_gather_dtype == torch.bfloat16
    got, want = _gather_full(model), dict(ref.named_parameters())
    for k in want:
        assert torch.equal(got[k].view(torch.int32), want[k].detach().view(torch.int32)), k


def test_module_api_and_states():
    from yafsdp_amd import fully_shard
    from yafsdp_amd.fully_shard import YaFSDPModule

    model = _wrap(_make(2), mp_policy=MP)
    assert isinstance(model, YaFSDPModule) and type(model).__name__ == "YaFSDPNet"
    assert isinstance(model.blocks[0], YaFSDPModule)
    with pytest.raises(AssertionError, match="deepcopy"):
        copy.deepcopy(model)
    with pytest.raises(ValueError, match="containers"):
        fully_shard(nn.ModuleList([nn.Linear(2, 2)]))
    with pytest.raises(AssertionError, match="already"):
        fully_shard(model.blocks[0])
    x = torch.randn(4, 128, device=DEV)
    model(x).float().sum().backward()  # the first pass through the root allocates the shared buffers
    # explicit unshard / reshard
    blk = model.blocks[1]
    handle = blk.unshard(async_op=True)
    handle.wait()
    assert blk.up.weight.dtype == torch.bfloat16 and blk.up.weight.shape == (256, 128)
    blk.reshard()
    assert blk.up.weight.dtype == torch.float32 and isinstance(blk.up.weight, RaggedShardDTensor)
    # the last user of each data buffer keeps its parameters unsharded after forward
    model(x)
    groups = [m._get_fsdp_state()._fsdp_param_group for m in [*model.blocks, model.norm]]
    assert [g.is_unsharded for g in groups] == [False, False, True, True]
    for m in (model.blocks[2], model.norm):
        m.reshard()  # a forward without a backward leaves them holding both data buffers
    model.set_reshard_after_forward(True)
    model(x)
    assert all(g.is_sharded for g in groups)
    with pytest.raises(ValueError):
        model.set_reshard_after_forward("yes")
    with pytest.raises(ValueError):
        model.set_modules_to_forward_prefetch([nn.Linear(2, 2)])
    model.blocks[0].set_modules_to_forward_prefetch([model.blocks[1]])
    model.blocks[2].set_modules_to_backward_prefetch([model.blocks[1]])
    model(x).float().sum().backward()
    torch.cuda.synchronize()
    assert all(p.grad is not None for p in model.parameters())


def test_nested_groups_must_not_share_a_buffer():
    from yafsdp_amd import fully_shard

    model = _make(5)
    for b in model.blocks:
        fully_shard(b, mp_policy=MP)
    fully_shard(model, mp_policy=MP)  # the root now owns `norm` and stays unsharded while its children run
    with pytest.raises(RuntimeError, match="share a (data|grad) buffer"):
        model(torch.randn(2, 128, device=DEV))  # ya_fsdp/_state.py:375-384


def test_lazy_init_requires_root_first():
    model = _wrap(_make(3), mp_policy=MP)
    with pytest.raises(RuntimeError, match="root module first"):
        model.blocks[0](torch.randn(2, 128, device=DEV))
        model(torch.randn(2, 128, device=DEV))


def test_logical_world_size_gives_each_rank_its_ragged_shard():
    from yafsdp_amd import fully_shard

    model0 = _make(4)
    full = torch.cat([p.detach().view(-1) for p in model0.blocks[0].parameters()])
    numels = [p.numel() for p in model0.blocks[0].parameters()]
    w = 3
    lay = make_layout(numels, w, 8)
    pieces = []
    for r in range(w):
        blk = copy.deepcopy(model0.blocks[0])
        fully_shard(blk, mesh=(w, r), mp_policy=MP)
        sharded = list(blk.parameters())
        assert [loc(p).numel() for p in sharded] == lay.sharded_numels(r)
        assert [p.placements[0].global_offset for p in sharded] == lay.global_offsets(r)
        pieces.append(torch.cat([loc(p) for p in sharded]))
    assert torch.equal(torch.cat(pieces), full)  # the ranks' fragments tile the flat parameter space


def test_list_of_modules_forms_one_group():
    """``fully_shard([a, b])``: one parameter group gathered before the first of the modules runs and released
    after the last (ya_fsdp/_state.py:575-613); training matches wrapping the same modules one by one."""
    from yafsdp_amd import fully_shard
    from yafsdp_amd.fully_shard import YaFSDPModule
    from yafsdp_amd.optim import fsdp_param_groups

    model0 = _make(31)
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(40 + s)) for s in range(3)]

    def train(grouped: bool):
        model = copy.deepcopy(model0)
        if grouped:
            out = fully_shard([model.blocks[0], model.blocks[1], model.blocks[0].up], mp_policy=MP)  # nested one dropped
            assert isinstance(out, list) and isinstance(model.blocks[0], YaFSDPModule) and isinstance(model.blocks[1], YaFSDPModule)
            assert not isinstance(model.blocks[0].up, YaFSDPModule)
        else:
            fully_shard(model.blocks[0], mp_policy=MP)
            fully_shard(model.blocks[1], mp_policy=MP)
        fully_shard(model.blocks[2], mp_policy=MP)
        fully_shard(model.norm, mp_policy=MP)
        fully_shard(model, mp_policy=MP)
        groups = fsdp_param_groups(model)
        assert len(groups) == (3 if grouped else 4)
        if grouped:
            assert len(groups[0].fsdp_params) == 6 and groups[0].modules == (model.blocks[0], model.blocks[1])
        opt = torch.optim.SGD(model.parameters(), lr=0.05)
        for x in xs:
            model(x).float().pow(2).mean().backward()
            if grouped:
                assert groups[0].is_sharded and not model._get_fsdp_state()._modules_to_run_forward
            opt.step()
            opt.zero_grad(set_to_none=True)
        torch.cuda.synchronize()
        return _gather_full(model)

    a, b = train(True), train(False)
    assert set(a) == set(b)
    for k in a:
        assert torch.equal(a[k].view(torch.int32), b[k].view(torch.int32)), k
    with pytest.raises(RuntimeError, match="single root"):
        m = _make(32)
        fully_shard([m.blocks[0], m.blocks[1]], mp_policy=MP)
        m.blocks[0](xs[0])


def test_state_dict_sees_sharded_parameters_even_when_unsharded():
    """ya_fsdp/_param_group.py:886-909: state_dict() / load_state_dict() first put the sharded parameters back."""
    model = _wrap(_make(41), mp_policy=MP)
    x = torch.randn(4, 128, device=DEV)
    model(x)  # forward only: the last users of the data buffers stay unsharded
    blk = model.blocks[2]
    assert blk.up.weight.dtype == torch.bfloat16 and blk.up.weight.dim() == 2
    sd = model.state_dict()
    assert all(v.dtype == torch.float32 and isinstance(v, RaggedShardDTensor) for v in sd.values())
    assert blk.up.weight.dtype == torch.float32  # swapped back by the hook
    new = {k: torch.zeros_like(v).fill_(0.25) for k, v in sd.items()}
    # the hook swaps the registered parameters only; the buffers are handed back by reshard(), as after any
    # forward without backward
    for m in (model.blocks[2], model.norm):
        m.reshard()
    model(x)
    assert blk.up.weight.dtype == torch.bfloat16
    model.load_state_dict(new)  # pre-hook: the load goes into the sharded masters
    assert blk.up.weight.dtype == torch.float32
    for m in (model.blocks[2], model.norm):
        m.reshard()
    group = blk._get_fsdp_state()._fsdp_param_group
    assert float(group._padded_sharded_param_data[None][: group.layout.total_numel].min()) == 0.25


def test_custom_gradient_buffer_assignment():
    """ya_fsdp/_state.py:127-136, 617-660: a group -> buffer-context index map replaces the round-robin
    assignment of the gradient buffers (accepted together with allow_no_grad_reduce, as in the reference)."""
    model0 = _make(8)
    xs = [torch.randn(16, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(90 + s)) for s in range(3)]
    ref = _reference_steps(model0, xs, lr=0.05)
    model = _wrap(copy.deepcopy(model0), mp_policy=MP)
    groups = [m._get_fsdp_state()._fsdp_param_group for m in (*model.blocks, model.norm)]
    model._get_fsdp_state()._lazy_init(
        allow_no_grad_reduce=True,
        param_group_to_grad_buffer_ctx_idx={groups[0]: 0, groups[1]: 1, groups[2]: 0, groups[3]: 1},
    )
    assert groups[0].grad_buffer_ctx is groups[2].grad_buffer_ctx
    assert groups[1].grad_buffer_ctx is groups[3].grad_buffer_ctx
    assert groups[0].grad_buffer_ctx is not groups[1].grad_buffer_ctx
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    for x in xs:
        model(x).float().pow(2).mean().backward()
        opt.step()
        opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    got, want = _gather_full(model), dict(ref.named_parameters())
    for k in want:
        assert torch.equal(got[k].view(torch.int32), want[k].detach().view(torch.int32)), k
    # without allow_no_grad_reduce the default is one shared buffer and a map is refused (:659-660)
    other = _wrap(copy.deepcopy(model0), mp_policy=MP)
    g2 = [m._get_fsdp_state()._fsdp_param_group for m in (*other.blocks, other.norm)]
    with pytest.raises(AssertionError):
        other._get_fsdp_state()._lazy_init(param_group_to_grad_buffer_ctx_idx={g: 0 for g in g2})


def _train(model, xs, lr, after_step=None):
    opt = torch.optim.SGD(model.parameters(), lr=lr)
    for x in xs:
        model(x).float().pow(2).mean().backward()
        opt.step()
        opt.zero_grad(set_to_none=True)
        if after_step is not None:
            after_step()
    torch.cuda.synchronize()
    return _gather_full(model)


def _assert_same_masters(got, want):
    assert set(got) == set(want)
    for k in want:
        assert torch.equal(got[k].view(torch.int32), want[k].detach().view(torch.int32)), k


def test_setters_that_must_not_change_the_numbers(monkeypatch):
    """ya_fsdp/fully_shard.py:138-239: keeping parameters unsharded after backward, forcing SUM (at world size 1
    no division either way, ya_fsdp/_collectives.py:221-267), a post-optimizer event for the all-gather stream to
    wait on, and explicit prefetch orders leave the training bit-identical."""
    model0 = _make(51)
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(60 + s)) for s in range(3)]
    want = dict(_reference_steps(model0, xs, lr=0.05).named_parameters())

    model = _wrap(copy.deepcopy(model0), mp_policy=MP)
    for m in (*model.blocks, model.norm):
        m.set_force_sum_reduction_for_comms(True)
    _assert_same_masters(_train(model, xs, 0.05), want)

    model = _wrap(copy.deepcopy(model0), mp_policy=MP)

    def mark():  # what a trainer does after optimizer.step(): the next all-gather waits for it
        model.set_post_optim_event(torch.cuda.current_stream().record_event())

    _assert_same_masters(_train(model, xs, 0.05, after_step=mark), want)

    model = _wrap(copy.deepcopy(model0), mp_policy=MP)
    blocks = list(model.blocks)
    blocks[0].set_modules_to_forward_prefetch([blocks[1]])
    blocks[1].set_modules_to_forward_prefetch([blocks[2]])
    blocks[2].set_modules_to_backward_prefetch([blocks[1]])
    blocks[1].set_modules_to_backward_prefetch([blocks[0]])
    _assert_same_masters(_train(model, xs, 0.05), want)

    # the library's own opt-in: reduce copy-in on the reduce-scatter stream (real autograd gradients here, freed
    # right after the launch that reads them on the other stream)
    model = _wrap(copy.deepcopy(model0), mp_policy=MP)
    model.set_reduce_copy_in_on_side_stream(True)
    groups = [g for m in model._fsdp_modules(True) if (g := m._get_fsdp_state()._fsdp_param_group) is not None]
    assert groups and all(g.reduce_copy_in_on_side_stream for g in groups)
    _assert_same_masters(_train(model, xs, 0.05), want)

    # the same through the environment, for a training script that cannot call the setter
    monkeypatch.setenv("YAFSDP_REDUCE_COPY_IN_ON_SIDE_STREAM", "1")
    model = _wrap(copy.deepcopy(model0), mp_policy=MP)
    monkeypatch.delenv("YAFSDP_REDUCE_COPY_IN_ON_SIDE_STREAM")
    groups = [g for m in model._fsdp_modules(True) if (g := m._get_fsdp_state()._fsdp_param_group) is not None]
    assert groups and all(g.reduce_copy_in_on_side_stream for g in groups)
    _assert_same_masters(_train(model, xs, 0.05), want)
    plain = _wrap(copy.deepcopy(model0), mp_policy=MP)
    assert not any(g.reduce_copy_in_on_side_stream
                   for m in plain._fsdp_modules(True) if (g := m._get_fsdp_state()._fsdp_param_group) is not None)



def test_parameters_kept_unsharded_between_micro_batches():
    """set_reshard_after_backward(False) for all but the last micro-batch of a step (every group on a data buffer
    of its own: reshard_after_forward=False): the second micro-batch finds the parameters gathered and skips the
    all-gather; the numbers equal those of the default schedule."""
    model0 = _make(53)
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(85 + s)) for s in range(4)]

    def run(keep: bool):
        model = _wrap(copy.deepcopy(model0), mp_policy=MP, reshard_after_forward=False)
        opt = torch.optim.SGD(model.parameters(), lr=0.05)
        groups = [m._get_fsdp_state()._fsdp_param_group for m in (*model.blocks, model.norm)]
        for i in range(0, 4, 2):
            if keep:
                model.set_reshard_after_backward(False)
            model(xs[i]).float().pow(2).mean().backward()
            if keep:
                assert all(g.is_unsharded for g in groups)
                model.set_reshard_after_backward(True)
            model(xs[i + 1]).float().pow(2).mean().backward()
            assert all(g.is_sharded for g in groups)
            opt.step()
            opt.zero_grad(set_to_none=True)
        torch.cuda.synchronize()
        return _gather_full(model)

    _assert_same_masters(run(True), run(False))


def test_custom_gradient_divide_factor():
    """set_gradient_divide_factor(4) at world size 1 copies the reduce buffer divided by 4 into the gradient shard
    (ya_fsdp/_collectives.py:140-148): with bf16 gradients the division by a power of two is exact, so the run
    equals plain training with a quarter of the learning rate... of the gradients that reach the masters."""
    model0 = _make(52)
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(80 + s)) for s in range(2)]
    model = _wrap(copy.deepcopy(model0), mp_policy=MP)
    for m in (*model.blocks, model.norm):
        m.set_gradient_divide_factor(4.0)
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    plain = _wrap(copy.deepcopy(model0), mp_policy=MP)
    opt_plain = torch.optim.SGD(plain.parameters(), lr=0.05)
    for x in xs[:1]:  # one step from identical masters: the gradients differ by exactly the factor
        model(x).float().pow(2).mean().backward()
        plain(x).float().pow(2).mean().backward()
        for p, q in zip(model.parameters(), plain.parameters()):
            assert torch.equal(loc(p.grad) * 4.0, loc(q.grad))
        opt.step(); opt_plain.step()
    torch.cuda.synchronize()


def test_frozen_and_tied_parameters():
    """A frozen parameter takes part in the all-gather but not in the reduce (ya_fsdp/_param_group.py:669-708,
    ya_fsdp/_collectives.py:166-170); a parameter registered on two modules is managed once and set on both
    (ya_fsdp/_init.py:150-189, ya_fsdp/_param.py:226-236)."""
    model0 = _make(61)
    model0.blocks[0].up.bias.requires_grad_(False)
    model0.blocks[1].down.weight.requires_grad_(False)
    model0.blocks[2].up.weight = model0.blocks[1].up.weight            # tied across two wrapped modules' parent
    model0.blocks[2].up.bias = model0.blocks[1].up.bias
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(95 + s)) for s in range(3)]
    want = dict(_reference_steps(model0, xs, lr=0.05).named_parameters())

    from yafsdp_amd import fully_shard

    model = copy.deepcopy(model0)
    assert model.blocks[2].up.weight is model.blocks[1].up.weight
    fully_shard(model.blocks[0], mp_policy=MP)
    fully_shard([model.blocks[1], model.blocks[2]], mp_policy=MP)       # the tie lives inside one group
    fully_shard(model.norm, mp_policy=MP)
    fully_shard(model, mp_policy=MP)
    params = list(model.parameters())
    assert len(params) == len(list(model0.parameters()))               # the tied pair counts once
    assert model.blocks[2].up.weight is model.blocks[1].up.weight
    frozen = [p for p in params if not p.requires_grad]
    assert len(frozen) == 2
    opt = torch.optim.SGD([p for p in params if p.requires_grad], lr=0.05)
    for x in xs:
        model(x).float().pow(2).mean().backward()
        assert all(p.grad is None for p in frozen)
        opt.step()
        opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    got = dict(model.named_parameters())  # world size 1: every sharded parameter is the whole flattened master
    assert set(got) == set(want)
    for k, v in want.items():
        assert torch.equal(loc(got[k]).view(v.shape).view(torch.int32), v.detach().view(torch.int32)), k


def test_ignored_parameters_stay_plain():
    """ignored_params (ya_fsdp/fully_shard.py:72, ya_fsdp/_init.py:123-189) are neither sharded nor cast: they
    keep their shape, dtype and ordinary autograd gradients."""
    from yafsdp_amd import fully_shard

    class Gained(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.Linear(128, 128)
            self.gain = nn.Parameter(torch.full((128,), 1.5))

        def forward(self, x):
            return self.lin(x) * self.gain.to(x.dtype)  # the module itself deals with the fp32 parameter

    torch.manual_seed(62)
    model = nn.Sequential(Gained(), Gained()).to(DEV)
    ignored = {model[0].gain, model[1].gain}
    for m in model:
        fully_shard(m, mp_policy=MP, ignored_params=ignored)
    fully_shard(model, mp_policy=MP)
    for m in model:
        group = m._get_fsdp_state()._fsdp_param_group
        assert len(group.fsdp_params) == 2  # weight and bias of the linear layer only
        assert m.gain.shape == (128,) and m.gain.dtype == torch.float32 and isinstance(m.gain, nn.Parameter)
    x = torch.randn(4, 128, device=DEV)
    model(x).float().pow(2).mean().backward()
    torch.cuda.synchronize()
    for m in model:
        assert m.gain.grad is not None and m.gain.grad.shape == (128,) and m.gain.grad.dtype == torch.float32
        assert m.gain.dim() == 1 and m.gain.numel() == 128
    assert all(p.grad is not None for p in model.parameters())


def test_profiler_ranges_appear_only_while_a_profiler_runs():
    """The reference's record_function ranges (ya_fsdp/_param_group.py:563, 669, 710, 740) are opened while a torch
    profiler is running, and skipped otherwise."""
    from torch.profiler import ProfilerActivity, profile

    from yafsdp_amd._common import _NO_RANGE, profiler_range

    assert profiler_range("x") is _NO_RANGE
    model = _wrap(_make(71), mp_policy=MP)
    x = torch.randn(4, 128, device=DEV)
    model(x).float().sum().backward()
    with profile(activities=[ProfilerActivity.CPU]) as prof:
        assert profiler_range("x") is not _NO_RANGE
        model(x).float().sum().backward()
        torch.cuda.synchronize()
    names = {e.name for e in prof.events()}
    for want in ("YaFSDP::all_gather", "YaFSDP::pre_forward", "YaFSDP::post_forward", "YaFSDP::pre_backward",
                 "YaFSDP::post_backward_reduce"):
        assert any(n.startswith(want) for n in names), (want, sorted(n for n in names if "FSDP" in n))
    assert profiler_range("x") is _NO_RANGE


def test_activation_checkpointing_recomputes_through_the_hooks():
    """Blocks run under torch.utils.checkpoint (non-reentrant): their forward is recomputed during backward, so the
    forward hooks fire again while the group is in its backward states (ya_fsdp/_state.py:301-345,
    ya_fsdp/_param_group.py:550-560).  The masters must come out as without checkpointing."""
    from torch.utils.checkpoint import checkpoint

    class CkptNet(Net):
        def forward(self, x):
            for b in self.blocks:
                x = checkpoint(b, x, use_reentrant=False)
            return self.norm(x)

    torch.manual_seed(81)
    plain0 = Net().to(DEV)
    ckpt0 = CkptNet().to(DEV)
    ckpt0.load_state_dict(plain0.state_dict())
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(120 + s),
                      requires_grad=True) for s in range(3)]
    want = _train(_wrap(plain0, mp_policy=MP), xs, 0.05)
    got = _train(_wrap(ckpt0, mp_policy=MP), xs, 0.05)
    _assert_same_masters(got, want)


def test_device_without_an_index_means_the_current_gpu():
    """fully_shard(device="cuda") and YaFSDPParamGroup / TensorTable with torch.device("cuda") resolve to the current
    GPU (tensors always report an indexed device)."""
    from yafsdp_amd import _native, fully_shard

    model = _make(3)
    x = torch.randn(4, 128, device=DEV)
    want = copy.deepcopy(model).to(torch.bfloat16)(x.to(torch.bfloat16))
    for b in model.blocks:
        fully_shard(b, mp_policy=MP, device="cuda")
    fully_shard(model.norm, mp_policy=MP, device=torch.device("cuda"))
    fully_shard(model, mp_policy=MP, device="cuda")
    got = model(x)
    assert torch.equal(got, want)
    got.float().pow(2).mean().backward()
    table = _native.TensorTable([8, 24], 32, torch.device("cuda"))
    flat = torch.zeros(32, dtype=torch.bfloat16, device=DEV)
    table.gather_in([torch.ones(8, dtype=torch.bfloat16, device=DEV), torch.ones(24, dtype=torch.bfloat16, device=DEV)],
                    flat, None, None, True)
    assert float(flat.float().sum()) == 32.0
    table.close()


def test_meta_device_model_is_materialised_empty_and_trains_after_initialisation():
    """Deferred initialisation as in ya_fsdp/_init.py:205-211: parameters on the meta device become uninitialised
    device tensors; the caller initialises the sharded parameters afterwards."""
    from yafsdp_amd import fully_shard

    ref = _make(9)
    with torch.device("meta"):
        model = Net()
    for b in model.blocks:
        fully_shard(b, mp_policy=MP, device=DEV)
    fully_shard(model.norm, mp_policy=MP, device=DEV)
    fully_shard(model, mp_policy=MP, device=DEV)
    assert all(p.device == DEV for p in model.parameters())
    with torch.no_grad():
        for p, q in zip(model.parameters(), ref.parameters()):
            p.copy_(q.reshape(p.shape))
    x = torch.randn(4, 128, device=DEV)
    want = copy.deepcopy(ref).to(torch.bfloat16)(x.to(torch.bfloat16))
    assert torch.equal(model(x), want)


@pytest.mark.parametrize("impl", ["foreach", "fused"])
def test_torch_adamw_and_clip_grad_norm_on_the_sharded_parameters(impl):
    """torch's own optimizer (foreach and fused) and torch.nn.utils.clip_grad_norm_ reach the local fragments through
    the sharded parameters' dispatch list (ya_fsdp/_tensor.py:122-316): the same calls on plain copies of the
    fragments give the same bits."""
    model = _wrap(_make(61), mp_policy=MP)
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(300 + s)) for s in range(3)]
    model(xs[0]).float().pow(2).mean().backward()  # lazy init
    model.zero_grad(set_to_none=True)
    params = list(model.parameters())
    twins = [nn.Parameter(loc(p).clone()) for p in params]
    opt = torch.optim.AdamW(params, lr=1e-3, weight_decay=0.1, **{impl: True})
    topt = torch.optim.AdamW(twins, lr=1e-3, weight_decay=0.1, **{impl: True})
    for x in xs:
        (model(x).float().pow(2).mean() * 100.0).backward()
        for t, p in zip(twins, params):
            t.grad = loc(p.grad).clone()
        norm = torch.nn.utils.clip_grad_norm_(params, 0.05, foreach=True)
        tnorm = torch.nn.utils.clip_grad_norm_(twins, 0.05, foreach=True)
        assert torch.equal(norm, tnorm) and float(norm) > 0.05
        opt.step()
        topt.step()
        for t, p in zip(twins, params):
            assert torch.equal(loc(p).view(torch.int32), t.detach().view(torch.int32))
            assert torch.equal(loc(p.grad).view(torch.int32), t.grad.view(torch.int32))
        opt.zero_grad(set_to_none=True)
        topt.zero_grad(set_to_none=True)
    st = opt.state[params[0]]
    assert isinstance(st["exp_avg"], RaggedShardDTensor) and st["exp_avg"].shape == params[0].shape
    # the next forward sees the updated masters (torch's step went through the version counter of the flat shard)
    y = model(xs[0])
    twin_model = _make(61)
    with torch.no_grad():
        for q, t in zip(twin_model.parameters(), twins):
            q.copy_(t.view(q.shape))
    assert torch.equal(y, twin_model.to(torch.bfloat16)(xs[0].to(torch.bfloat16)))


def test_store_policy_follows_the_number_of_gradient_buffers(monkeypatch):
    """How much of a reduce buffer's end is stored write-through is chosen per parameter group when the root is
    initialised, from the number of gradient buffers that take turns (the tables of the group carry it); the
    process-wide options are the application's and stay as they are.  Either way the same bits (every other test)."""
    from yafsdp_amd import _native, fully_shard

    def tails(model):
        out = set()
        for state in model._get_fsdp_state()._state_ctx.all_states:
            if (group := state._fsdp_param_group) is not None:
                out |= {t.get_option(_native.OPT_GATHER_TAIL_MB) for t in group._tables.values()}
        return out

    x = torch.randn(4, 128, device=DEV)
    defaults = _native.get_store_policy()
    assert defaults == _native.STORE_POLICIES["rotating_sets"]  # the library's defaults
    model = _wrap(_make(61), mp_policy=MP)  # four groups, one gradient buffer
    model(x).float().pow(2).mean().backward()
    assert tails(model) == {128} and _native.get_store_policy() == defaults
    # a gradient buffer per group (gradient accumulation without reduction): four buffers take turns
    many = _wrap(_make(63), mp_policy=MP)
    many._get_fsdp_state()._lazy_init(allow_no_grad_reduce=True)
    many(x).float().pow(2).mean().backward()
    assert tails(many) == {64} and tails(model) == {128}  # two models in one process keep their own
    single = fully_shard(Block(128, 256).to(DEV), mp_policy=MP)  # one group
    single(x).float().pow(2).mean().backward()
    assert tails(single) == {128} and _native.get_store_policy() == defaults
    # the environment can leave everything alone, or make an explicit process-wide choice
    monkeypatch.setenv("YAFSDP_STORE_POLICY", "keep")
    _native.set_store_policy((1, 2, 3, 4))
    kept = _wrap(_make(62), mp_policy=MP)
    kept(x).float().pow(2).mean().backward()
    assert _native.get_store_policy() == (1, 2, 3, 4) and tails(kept) == {-1}
    monkeypatch.setenv("YAFSDP_STORE_POLICY", "single_set")
    fully_shard(Block(128, 256).to(DEV), mp_policy=MP)(x).float().pow(2).mean().backward()
    assert _native.get_store_policy() == _native.STORE_POLICIES["single_set"]
    monkeypatch.setenv("YAFSDP_STORE_POLICY", "fastest")
    with pytest.raises(ValueError, match="YAFSDP_STORE_POLICY"):
        fully_shard(Block(128, 256).to(DEV), mp_policy=MP)(x)
