"""Flat-shard optimizer passes on ``fully_shard`` modules (one GPU): the fused
AdamW step, gradient clipping and zero_grad run as one launch per parameter
group and match the C oracle bit for bit on the same gradients."""

import copy

import pytest
import torch
import torch.nn as nn

from oracle import cref

from helpers import assert_bits_equal, loc
from test_gpu_fully_shard import DEV, MP, Net, _make, _wrap

pytestmark = pytest.mark.gpu
HP = dict(lr=1e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)


def _groups(model):
    from yafsdp_amd.optim import fsdp_param_groups

    return fsdp_param_groups(model)


def _xs(n, seed=0, batch=8):
    return [torch.randn(batch, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(seed + s))
            for s in range(n)]


class _CpuMirror:
    """CPU copies of every group's flat master / moment buffers, stepped by the oracle."""

    def __init__(self, groups):
        self.p = [g._padded_sharded_param_data[None].detach().cpu().clone() for g in groups]
        self.m = [torch.zeros_like(p) for p in self.p]
        self.v = [torch.zeros_like(p) for p in self.p]

    def step(self, groups, step, grad_scale=None, **hp):
        outs = []
        for i, g in enumerate(groups):
            grad = g._padded_sharded_param_grad[None].detach().cpu().clone()
            out16 = torch.zeros(grad.numel(), dtype=torch.bfloat16)
            cref.adamw_step(self.p[i], grad, self.m[i], self.v[i], out16, lr=hp["lr"], beta1=hp["betas"][0],
                            beta2=hp["betas"][1], eps=hp["eps"], weight_decay=hp["weight_decay"], step=step,
                            grad_scale=grad_scale)
            outs.append(out16)
        return outs


def test_flat_adamw_matches_the_oracle_and_prefills_the_all_gather_input():
    from yafsdp_amd.optim import FlatAdamW

    model = _wrap(_make(7), mp_policy=MP)
    groups = _groups(model)
    assert len(groups) == 4
    opt = FlatAdamW(model.parameters(), **HP)
    mirror = _CpuMirror(groups)
    for step, x in enumerate(_xs(4), start=1):
        model(x).float().pow(2).mean().backward()
        outs = mirror.step(groups, step, **HP)
        opt.step()
        for g, p, o in zip(groups, mirror.p, outs):
            assert_bits_equal(g._padded_sharded_param_data[None], p, f"masters of {g} after step {step}")
            assert_bits_equal(g._all_gather_input[None], o, f"all-gather input of {g} after step {step}")
            assert None in g._all_gather_input_set_dtypes  # the next unshard skips its cast
        opt.zero_grad(set_to_none=True)
    for i, g in enumerate(groups):
        unit = [u for u in opt._units[0] if u.group is g][0]
        assert_bits_equal(unit.exp_avg, mirror.m[i], "exp_avg")
        assert_bits_equal(unit.exp_avg_sq, mirror.v[i], "exp_avg_sq")
    # state views alias the flat moments
    p0 = groups[0].fsdp_params[0].sharded_param
    assert loc(opt.state[p0]["exp_avg"]).data_ptr() == [u for u in opt._units[0] if u.group is groups[0]][0].exp_avg.data_ptr()
    assert opt.state[p0]["exp_avg"].shape == p0.shape  # shaped (and wrapped) like the sharded parameter


def test_fused_copy_in_changes_nothing_downstream():
    """Same model, same inputs: with and without the fused copy-in the outputs and masters are bit-identical."""
    from yafsdp_amd.optim import FlatAdamW

    model0 = _make(8)
    outs = []
    for fuse in (True, False):
        model = _wrap(copy.deepcopy(model0), mp_policy=MP)
        opt = FlatAdamW(model.parameters(), fuse_copy_in=fuse, **HP)
        ys = []
        for x in _xs(3, seed=20):
            y = model(x)
            ys.append(y.detach().clone())
            y.float().pow(2).mean().backward()
            opt.step()
            opt.zero_grad(set_to_none=True)
        ys.append(torch.cat([g._padded_sharded_param_data[None] for g in _groups(model)]).bfloat16())
        outs.append(ys)
    for a, b in zip(*outs):
        assert_bits_equal(a, b, "fused vs unfused copy-in")


def test_clip_grad_norm_matches_the_oracle_and_torch():
    from yafsdp_amd.optim import clip_grad_norm_, grad_clip_coef

    model = _wrap(_make(9), mp_policy=MP)
    groups = _groups(model)
    (model(_xs(1, seed=30)[0]).float().pow(2).mean() * 50.0).backward()
    grads = [g._padded_sharded_param_grad[None].detach().cpu().clone() for g in groups]
    total = sum(cref.sumsq(x) for x in grads)
    for max_norm in (1e-3, 1e9):
        norm, coef = cref.clip_coef(total, max_norm)
        n_dev, c_dev = grad_clip_coef(model, max_norm)
        assert abs(n_dev.item() - norm) <= 6e-8 * norm and abs(c_dev.item() - coef) <= 1.2e-7 * coef
        # torch's own clipping on copies of the per-parameter gradients
        tparams = [nn.Parameter(loc(p).clone()) for p in model.parameters()]
        for tp, p in zip(tparams, model.parameters()):
            tp.grad = loc(p.grad).clone()
        tnorm = torch.nn.utils.clip_grad_norm_(tparams, max_norm)
        got_norm = clip_grad_norm_(model, max_norm)
        assert abs(got_norm.item() - tnorm.item()) <= 2e-6 * tnorm.item()
        coef_used = c_dev.item()
        for g, x in zip(groups, grads):
            want = x.clone()
            cref.flat_scale(want, coef_used)
            assert_bits_equal(g._padded_sharded_param_grad[None], want, f"clipped grads max_norm={max_norm}")
        for tp, p in zip(tparams, model.parameters()):
            torch.testing.assert_close(loc(p.grad), tp.grad, rtol=3e-6, atol=0)
        grads = [g._padded_sharded_param_grad[None].detach().cpu().clone() for g in groups]
        total = sum(cref.sumsq(x) for x in grads)
    assert coef_used == 1.0  # nothing clipped at 1e9: gradients untouched


def test_grad_scale_fused_into_the_step_equals_clip_then_step():
    from yafsdp_amd.optim import FlatAdamW, clip_grad_norm_, grad_clip_coef

    model0 = _make(10)
    x = _xs(1, seed=40)[0]
    results = []
    for fused in (True, False):
        model = _wrap(copy.deepcopy(model0), mp_policy=MP)
        opt = FlatAdamW(model.parameters(), **HP)
        for _ in range(2):
            (model(x).float().pow(2).mean() * 10).backward()
            if fused:
                _, coef = grad_clip_coef(model, 0.05)
                opt.step(grad_scale=coef, zero_grad=True)
                assert all(float(g._padded_sharded_param_grad[None].abs().max()) == 0.0 for g in _groups(model))
            else:
                clip_grad_norm_(model, 0.05)
                opt.step()
            opt.zero_grad(set_to_none=True)
        results.append(torch.cat([g._padded_sharded_param_data[None] for g in _groups(model)]))
    assert_bits_equal(results[0], results[1], "fused gradient scale")


def test_partial_gradients_and_ragged_fragments():
    """Logical world size 3: fragments start at odd offsets; one parameter is frozen, one has no gradient."""
    from yafsdp_amd import fully_shard
    from yafsdp_amd.optim import FlatAdamW, clip_grad_norm_

    torch.manual_seed(11)
    blk = Net(layers=1).to(DEV)
    blk.blocks[0].up.bias.requires_grad_(False)
    fully_shard(blk.blocks[0], mesh=(3, 1), mp_policy=MP, shard_alignment=1)
    fully_shard(blk.norm, mesh=(3, 1), mp_policy=MP, shard_alignment=1)
    fully_shard(blk, mesh=(3, 1), mp_policy=MP, shard_alignment=1)
    groups = _groups(blk)
    opt = FlatAdamW([p for p in blk.parameters() if p.requires_grad], **HP)
    blk(_xs(1, seed=50)[0]).float().pow(2).mean().backward()
    g0 = groups[0]
    with_grad = [fp for fp in g0.fsdp_params if fp.requires_grad]
    with_grad[0].sharded_param.grad = None  # as if this parameter had not taken part in the step
    before = [g._padded_sharded_param_data[None].detach().cpu().clone() for g in groups]
    grads = [g._padded_sharded_param_grad[None].detach().cpu().clone() for g in groups]
    clip_grad_norm_(blk, 1e-4)
    # oracle: norm over the fragments that have a gradient only
    pos, total = 0, 0.0
    frag = []
    for gi, g in enumerate(groups):
        pos = 0
        for fp, n in zip(g.fsdp_params, g._sharded_param_numels[None]):
            has = fp.requires_grad and fp.sharded_param.grad is not None
            frag.append((gi, pos, n, has))
            if has:
                total += cref.sumsq(grads[gi][pos : pos + n].clone())
            pos += n
    norm, coef = cref.clip_coef(total, 1e-4)
    opt.step()
    for gi, pos, n, has in frag:
        p = before[gi][pos : pos + n].clone()
        if has and n:
            gr = grads[gi][pos : pos + n].clone()
            cref.flat_scale(gr, coef)
            cref.adamw_step(p, gr, torch.zeros(n), torch.zeros(n), None, lr=HP["lr"], beta1=0.9, beta2=0.95,
                            eps=1e-8, weight_decay=0.1, step=1)
        assert_bits_equal(groups[gi]._padded_sharded_param_data[None][pos : pos + n], p, f"fragment {gi}:{pos}+{n}")
    assert None not in g0._all_gather_input_set_dtypes  # partial pass: the next forward casts the shard itself


def test_state_dict_round_trip_continues_bit_identically():
    from yafsdp_amd.optim import FlatAdamW

    model0 = _make(12)
    xs = _xs(4, seed=60)

    def run(split):
        model = _wrap(copy.deepcopy(model0), mp_policy=MP)
        opt = FlatAdamW(model.parameters(), **HP)
        for i, x in enumerate(xs):
            if split and i == 2:
                sd = copy.deepcopy(opt.state_dict())
                assert sd["state"][0]["step"].item() == 2.0
                opt = FlatAdamW(model.parameters(), **HP)
                opt.load_state_dict(sd)
            model(x).float().pow(2).mean().backward()
            opt.step()
            opt.zero_grad(set_to_none=True)
        return torch.cat([g._padded_sharded_param_data[None] for g in _groups(model)])

    assert_bits_equal(run(True), run(False), "resume from a state dict")


def test_zero_grad_and_stale_copy_guard():
    from yafsdp_amd.optim import FlatAdamW, zero_grad

    model = _wrap(_make(13), mp_policy=MP)
    opt = FlatAdamW(model.parameters(), **HP)
    x = _xs(1, seed=70)[0]
    model(x).float().pow(2).mean().backward()
    opt.step()
    zero_grad(model)
    for p in model.parameters():
        assert p.grad is not None and float(loc(p.grad).abs().max()) == 0.0
    # a torch op changes the masters after the fused step: the next forward must cast again
    g = _groups(model)[0]
    with torch.no_grad():
        g.fsdp_params[0].sharded_param.mul_(2.0)
    model(x)
    torch.cuda.synchronize()
    assert_bits_equal(g._all_gather_input[None], g._padded_sharded_param_data[None].bfloat16(), "stale copy replaced")


def test_plain_parameters_and_errors():
    from yafsdp_amd.optim import FlatAdamW, clip_grad_norm_

    w = nn.Parameter(torch.randn(1000, device=DEV))
    opt = FlatAdamW([w], **HP)
    w.grad = torch.randn(1000, device=DEV)
    p, gr = w.detach().cpu().clone(), w.grad.cpu().clone()
    opt.step()
    cref.adamw_step(p, gr, torch.zeros(1000), torch.zeros(1000), None, lr=HP["lr"], beta1=0.9, beta2=0.95, eps=1e-8,
                    weight_decay=0.1, step=1)
    assert_bits_equal(w.detach(), p, "plain parameter")
    with pytest.raises(TypeError):
        FlatAdamW([nn.Parameter(torch.zeros(4, device=DEV, dtype=torch.bfloat16))], **HP).step()
    with pytest.raises(ValueError):
        clip_grad_norm_(nn.Linear(2, 2).to(DEV), 1.0)
    with pytest.raises(NotImplementedError):
        clip_grad_norm_(_wrap(_make(14), mp_policy=MP), 1.0, norm_type=1.0)


def test_fused_grad_norm_matches_the_read_pass():
    """enable_fused_grad_norm: the post-reduce leaves the squared norm of every gradient shard; grad_clip_coef adds
    those sums up and reads a shard again only when they no longer describe its gradients."""
    from yafsdp_amd import _native
    from yafsdp_amd.optim import (disable_fused_grad_norm, enable_fused_grad_norm, fsdp_param_groups,
                                  grad_clip_coef, zero_grad)

    model = _wrap(_make(41), mp_policy=MP)
    x = torch.randn(8, 128, device=DEV)
    model(x).float().pow(2).mean().backward()  # lazy init
    zero_grad(model)
    model.zero_grad(set_to_none=True)
    enable_fused_grad_norm(model)
    groups = fsdp_param_groups(model)
    calls = {"read": 0}
    real = _native.sumsq_partials

    def counting(*a, **k):
        calls["read"] += 1
        return real(*a, **k)

    _native.sumsq_partials = counting
    try:
        model(x).float().pow(2).mean().backward()
        assert all(g._grad_sumsq_token.get(None) is not None for g in groups)
        norm_fused, coef_fused = grad_clip_coef(model, 1e-3)
        assert calls["read"] == 0                      # every sum came from the post-reduce
        disable_fused_grad_norm(model)
        norm_read, coef_read = grad_clip_coef(model, 1e-3)
        assert calls["read"] == len(groups)
        assert torch.allclose(norm_fused, norm_read, rtol=2e-7, atol=0) and float(norm_read) > 0
        assert torch.allclose(coef_fused, coef_read, rtol=2e-7, atol=0)
        # a torch op on one gradient: that group, and only that group, is read again
        enable_fused_grad_norm(model)
        model.zero_grad(set_to_none=True)
        model(x).float().pow(2).mean().backward()
        calls["read"] = 0
        next(iter(model.blocks[1].parameters())).grad.mul_(3.0)
        norm_a, _ = grad_clip_coef(model, 1e-3)
        assert calls["read"] == 1
        disable_fused_grad_norm(model)
        norm_b, _ = grad_clip_coef(model, 1e-3)
        assert torch.allclose(norm_a, norm_b, rtol=2e-7, atol=0) and float(norm_b) > float(norm_read)
        # gradient accumulation: the second reduce adds into the shard and its sums describe the total
        enable_fused_grad_norm(model)
        model(x).float().pow(2).mean().backward()
        calls["read"] = 0
        norm_c, _ = grad_clip_coef(model, 1e-3)
        assert calls["read"] == 0
        disable_fused_grad_norm(model)
        norm_d, _ = grad_clip_coef(model, 1e-3)
        assert torch.allclose(norm_c, norm_d, rtol=2e-7, atol=0)
        # set_to_none: no gradients, nothing to add up from stale sums
        enable_fused_grad_norm(model)
        model.zero_grad(set_to_none=True)
        model(x).float().pow(2).mean().backward()
        model.blocks[0].zero_grad(set_to_none=True)
        calls["read"] = 0
        norm_e, _ = grad_clip_coef(model, 1e-3)
        disable_fused_grad_norm(model)
        norm_f, _ = grad_clip_coef(model, 1e-3)
        assert torch.allclose(norm_e, norm_f, rtol=2e-7, atol=0) and float(norm_f) < float(norm_read)
    finally:
        _native.sumsq_partials = real
        disable_fused_grad_norm(model)


def test_training_with_fused_grad_norm_equals_training_without():
    from yafsdp_amd.optim import FlatAdamW, enable_fused_grad_norm, grad_clip_coef

    model0 = _make(42)
    xs = [torch.randn(8, 128, device=DEV, generator=torch.Generator(device=DEV).manual_seed(300 + s)) for s in range(4)]

    def run(fused: bool):
        model = _wrap(copy.deepcopy(model0), mp_policy=MP)
        opt = FlatAdamW(model.parameters(), lr=1e-2, weight_decay=0.1)
        norms = []
        for i, x in enumerate(xs):
            model(x).float().pow(2).mean().backward()
            if fused and i == 0:
                enable_fused_grad_norm(model)  # after the first backward: the groups exist and hold gradients
            norm, coef = grad_clip_coef(model, 0.05)
            norms.append(float(norm))
            opt.step(grad_scale=coef)
            opt.zero_grad(set_to_none=True)
        torch.cuda.synchronize()
        return norms, [loc(p).clone() for p in model.parameters()]

    n1, p1 = run(True)
    n0, p0 = run(False)
    assert n1 == pytest.approx(n0, rel=3e-7)
    for a, b in zip(p1, p0):
        assert torch.allclose(a, b, rtol=0, atol=2e-7)


def test_fused_grad_norm_falls_back_when_the_reduce_writes_the_shard_directly():
    """Without mixed precision a size-1 group reduces straight into the gradient shard
    (ya_fsdp/_collectives.py:112-125): no post-reduce runs, so the norm is read from the shards as before."""
    from yafsdp_amd.optim import disable_fused_grad_norm, enable_fused_grad_norm, fsdp_param_groups, grad_clip_coef

    model = _wrap(_make(43))
    x = torch.randn(8, 128, device=DEV)
    model(x).pow(2).mean().backward()
    enable_fused_grad_norm(model)
    model.zero_grad(set_to_none=True)
    model(x).pow(2).mean().backward()
    assert all(g._grad_sumsq_token.get(None) is None for g in fsdp_param_groups(model))
    norm_a, _ = grad_clip_coef(model, 1.0)
    disable_fused_grad_norm(model)
    norm_b, _ = grad_clip_coef(model, 1.0)
    want = torch.sqrt(sum(loc(p.grad).double().pow(2).sum() for p in model.parameters())).float()
    assert torch.allclose(norm_a, norm_b, rtol=2e-7, atol=0) and torch.allclose(norm_b, want, rtol=1e-6, atol=0)


def test_fused_grad_norm_small_group_with_a_frozen_parameter_in_the_middle():
    """A group of three 512-element parameters whose middle one is frozen: its gradient shard has two disjoint
    ranges, more than the one tile its post-reduce covers.  The read pass must find room for both."""
    from yafsdp_amd import fully_shard
    from yafsdp_amd.optim import disable_fused_grad_norm, enable_fused_grad_norm, fsdp_param_groups, grad_clip_coef

    class Tiny3(nn.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(5)
            self.a = nn.Parameter(torch.randn(512, generator=g))
            self.b = nn.Parameter(torch.randn(512, generator=g), requires_grad=False)
            self.c = nn.Parameter(torch.randn(512, generator=g))

        def forward(self, x):
            return (x * self.a + self.b) * self.c

    model = fully_shard(Tiny3().to(DEV), mp_policy=MP)
    x = torch.randn(4, 512, device=DEV)
    model(x).float().pow(2).mean().backward()
    (group,) = fsdp_param_groups(model)
    assert group._padded_sharded_param_grad[None].numel() <= 4096
    enable_fused_grad_norm(model)
    try:
        assert group._grad_sumsq_slot[None][1] - group._grad_sumsq_slot[None][0] >= 2
        model.zero_grad(set_to_none=True)
        model(x).float().pow(2).mean().backward()
        norm_fused, coef_fused = grad_clip_coef(model, 1e-3)   # two ranges: read pass into the group's slot
        norm_again, _ = grad_clip_coef(model, 1e-3)            # and again over the same slot
    finally:
        disable_fused_grad_norm(model)
    norm_read, coef_read = grad_clip_coef(model, 1e-3)
    want = torch.sqrt(sum(loc(p.grad).double().pow(2).sum() for p in model.parameters() if p.grad is not None)).float()
    assert float(norm_read) > 0 and torch.allclose(norm_read, want, rtol=1e-6, atol=0)
    assert torch.equal(norm_fused, norm_read) and torch.equal(norm_again, norm_read) and torch.equal(coef_fused, coef_read)


def test_fused_grad_norm_slot_is_clean_after_a_read_pass_left_more_sums():
    """Three trainable 512-element parameters: an iteration whose middle gradient is dropped goes through the read
    pass and leaves two sums in the group's slot; the next iteration's post-reduce writes one.  The second sum must
    not be counted again."""
    from yafsdp_amd import fully_shard
    from yafsdp_amd.optim import disable_fused_grad_norm, enable_fused_grad_norm, grad_clip_coef

    class Tiny3(nn.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(6)
            self.a = nn.Parameter(torch.randn(512, generator=g))
            self.b = nn.Parameter(torch.randn(512, generator=g))
            self.c = nn.Parameter(torch.randn(512, generator=g))

        def forward(self, x):
            return (x * self.a + self.b) * self.c

    model = fully_shard(Tiny3().to(DEV), mp_policy=MP)
    x = torch.randn(4, 512, device=DEV)
    model(x).float().pow(2).mean().backward()
    enable_fused_grad_norm(model)
    try:
        model.zero_grad(set_to_none=True)
        model(x).float().pow(2).mean().backward()
        model.b.grad = None                       # two ranges: read pass, two sums in the slot
        grad_clip_coef(model, 1e-3)
        model.zero_grad(set_to_none=True)
        model(x).float().pow(2).mean().backward()  # all three gradients: the post-reduce's own single sum
        norm_fused, _ = grad_clip_coef(model, 1e-3)
    finally:
        disable_fused_grad_norm(model)
    norm_read, _ = grad_clip_coef(model, 1e-3)
    assert float(norm_read) > 0 and torch.equal(norm_fused, norm_read)
