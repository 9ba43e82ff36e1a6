"""Randomised parity of the buffer-path kernels against the oracle (hypothesis, derandomised: the same
examples on every run).  Shapes, dtypes, alignments, factors and per-tensor modes are drawn together, which
reaches combinations the parametrised tests do not enumerate.  Each example is small; every one names itself
on stdout before it touches the GPU."""

import os

import numpy as np
import pytest
import torch
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

from oracle import torch_ops

from helpers import DTYPES, assert_bits_equal, mixed_values

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
FACTORS = [None, 1.0, 2.0, 3.0, 8.0, 0.5, 1000.0, 64.0]
# YAFSDP_PROPERTY_SCALE=k draws k times as many examples, and fresh ones on every run (a longer search by hand; the
# default is the fixed set)
SCALE = max(1, int(os.environ.get("YAFSDP_PROPERTY_SCALE", "1")))
COMMON = dict(deadline=None, derandomize=SCALE == 1, suppress_health_check=list(HealthCheck), print_blob=SCALE > 1)


@pytest.fixture(scope="module")
def nat():
    from yafsdp_amd import _native

    return _native


def _view_at(x: torch.Tensor, offset: int, fill: float = 3.0) -> tuple[torch.Tensor, torch.Tensor]:
    """A device copy of ``x`` that starts ``offset`` elements into its allocation, with guard lanes around it."""
    buf = torch.full((x.numel() + offset + 9,), fill, dtype=x.dtype, device=DEV)
    view = buf[offset : offset + x.numel()]
    view.copy_(x)
    return buf, view


tables = st.lists(st.one_of(st.just(0), st.integers(1, 40), st.integers(1, 6000)), min_size=1, max_size=40)
# which stores write through (flat kernels, post-reduce, scatter-out tail, gather-in tail, in megabytes from the end
# of the output): the tables here are smaller than a megabyte, so every kind of kernel runs either all write-through
# or all non-temporal
ALL_MB = 1 << 20
policies = st.sampled_from([(ALL_MB, ALL_MB, 0, 96), (0, 0, 0, 128), (0, 0, 0, 0), (ALL_MB, ALL_MB, ALL_MB, ALL_MB)])


@settings(max_examples=120 * SCALE, **COMMON)
@given(src_dt=st.sampled_from(DTYPES), dst_dt=st.sampled_from(DTYPES), n=st.integers(0, 70_000),
       s_off=st.integers(0, 8), d_off=st.integers(0, 8), factor=st.sampled_from(FACTORS), acc=st.booleans(),
       seed=st.integers(0, 2**20), policy=policies)
def test_post_reduce_any_shape(nat, src_dt, dst_dt, n, s_off, d_off, factor, acc, seed, policy):
    nat.set_store_policy(policy)
    print("post_reduce", src_dt, dst_dt, n, s_off, d_off, factor, acc, seed, flush=True)
    g = torch.Generator().manual_seed(seed)
    chunk = mixed_values(g, n, src_dt, 1e-3)
    shard0 = mixed_values(g, n, dst_dt, 1e-4).flip(0).contiguous()
    want = shard0.clone()
    torch_ops.reduce_scatter_local(want, chunk.clone(), 1, 0, None, factor, "add" if acc else "copy")
    _, d_chunk = _view_at(chunk, s_off)
    buf, d_shard = _view_at(shard0, d_off)
    nat.post_reduce(d_shard, d_chunk, factor, acc)
    assert_bits_equal(d_shard, want, "shard")
    guard = torch.cat([buf[:d_off], buf[d_off + n :]]).float()
    assert float(guard.min()) == 3.0 and float(guard.max()) == 3.0




@settings(max_examples=80 * SCALE, **COMMON)
@given(numels=tables, pad=st.integers(0, 700), grad_dt=st.sampled_from(DTYPES), rs_dt=st.sampled_from(DTYPES),
       pre=st.sampled_from(FACTORS), two_waves=st.booleans(), zero_pad=st.booleans(), seed=st.integers(0, 2**20), policy=policies)
def test_gather_in_any_table(nat, numels, pad, grad_dt, rs_dt, pre, two_waves, zero_pad, seed, policy):
    nat.set_store_policy(policy)
    print("gather_in", numels, pad, grad_dt, rs_dt, pre, two_waves, zero_pad, seed, flush=True)
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    p, t = len(numels), sum(numels)
    t_pad = t + pad
    grads = [mixed_values(g, n, grad_dt, 1e-3) for n in numels]
    modes = rng.integers(0, 3, size=p).tolist()
    old = torch.zeros(t_pad + 8, dtype=rs_dt)
    old[:t_pad] = mixed_values(g, t_pad, rs_dt, 1e-3).flip(0)
    old[t_pad:] = 5.0
    want = old.clone()
    views = list(want[:t].split(numels))
    cp = [i for i, m in enumerate(modes) if m == 1]
    ad = [i for i, m in enumerate(modes) if m == 2]
    torch_ops.reduce_copy_in([views[i] for i in cp], [grads[i] for i in cp], False)
    torch_ops.reduce_copy_in([views[i] for i in ad], [grads[i] for i in ad], True)
    if zero_pad:
        want[t:t_pad] = 0
    torch_ops.div_if_needed(want[:t_pad], pre)
    default = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_TABLE_LARGE_LOG2, 0 if two_waves else default)
    try:
        table = nat.TensorTable(numels, t_pad, DEV)
    finally:
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default)
    got = old.to(DEV)
    dgrads = [_view_at(x, int(rng.integers(0, 8)))[1] for x in grads]
    table.gather_in(dgrads, got, modes, pre, zero_pad=zero_pad)
    assert_bits_equal(got, want, "reduce buffer")
    table.close()


@settings(max_examples=80 * SCALE, **COMMON)
@given(numels=tables, pad=st.integers(0, 700), flat_dt=st.sampled_from(DTYPES), out_dt=st.sampled_from(DTYPES),
       two_waves=st.booleans(), bound=st.booleans(), seed=st.integers(0, 2**20), tile_mode=st.integers(0, 2), policy=policies)
def test_scatter_out_any_table(nat, numels, pad, flat_dt, out_dt, two_waves, bound, seed, tile_mode, policy):
    nat.set_store_policy(policy)
    print("scatter_out", numels, pad, flat_dt, out_dt, two_waves, bound, seed, tile_mode, flush=True)
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    p, t = len(numels), sum(numels)
    flat = mixed_values(g, t + pad, flat_dt)
    modes = rng.integers(0, 2, size=p).tolist()
    offs = [int(rng.integers(0, 8)) for _ in numels]
    bufs, views = zip(*[_view_at(torch.full((n,), 3.0, dtype=out_dt), o) for n, o in zip(numels, offs)])
    default = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_TABLE_LARGE_LOG2, 0 if two_waves else default)
    nat.set_option(nat.OPT_SCATTER_TILE, tile_mode)  # 0 from the layout, 1 short tiles, 2 the gather-in tile
    try:
        table = nat.TensorTable(numels, t + pad, DEV)
    finally:
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default)
        nat.set_option(nat.OPT_SCATTER_TILE, 0)
    d_flat = flat.to(DEV)
    if bound:
        binding = table.bind(list(views), modes)
        binding.scatter_out(d_flat)
        binding.close()
    else:
        table.scatter_out(d_flat, list(views), modes)
    pos = 0
    for i, n in enumerate(numels):
        ref = torch.full((n + offs[i] + 9,), 3.0, dtype=out_dt)
        if modes[i]:
            ref[offs[i] : offs[i] + n].copy_(flat[pos : pos + n])
        assert_bits_equal(bufs[i], ref, f"tensor {i} with its guard lanes")
        pos += n
    table.close()


@settings(max_examples=80 * SCALE, **COMMON)
@given(numels=tables, pad=st.integers(0, 700), master_dt=st.sampled_from(DTYPES), param_dt=st.sampled_from(DTYPES),
       shard_n=st.integers(0, 9000), two_waves=st.booleans(), seed=st.integers(0, 2**20), tile_mode=st.integers(0, 2), policy=policies)
def test_copy_in_scatter_out_any_table(nat, numels, pad, master_dt, param_dt, shard_n, two_waves, seed, tile_mode, policy):
    nat.set_store_policy(policy)
    """Copy-in and copy-out as one launch: both halves with their guard lanes against the oracle."""
    print("copy_in_scatter_out", numels, pad, master_dt, param_dt, shard_n, two_waves, seed, tile_mode, flush=True)
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    p, t = len(numels), sum(numels)
    gathered = mixed_values(g, t + pad, param_dt)
    master = mixed_values(g, shard_n, master_dt)
    modes = rng.integers(0, 2, size=p).tolist()
    offs = [int(rng.integers(0, 8)) for _ in numels]
    bufs, views = zip(*[_view_at(torch.full((n,), 3.0, dtype=param_dt), o) for n, o in zip(numels, offs)])
    m_buf, m_view = _view_at(master, int(rng.integers(0, 4)))
    a_off = int(rng.integers(0, 8))
    a_buf, a_view = _view_at(torch.full((shard_n,), 3.0, dtype=param_dt), a_off)
    default = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_TABLE_LARGE_LOG2, 0 if two_waves else default)
    nat.set_option(nat.OPT_SCATTER_TILE, tile_mode)
    try:
        table = nat.TensorTable(numels, t + pad, DEV)
    finally:
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default)
        nat.set_option(nat.OPT_SCATTER_TILE, 0)
    assert table.copy_in_scatter_out(gathered.to(DEV), list(views), a_view, m_view, modes)
    want_ag = torch.full((shard_n + a_off + 9,), 3.0, dtype=param_dt)
    torch_ops.copy_in(want_ag[a_off : a_off + shard_n], master)
    assert_bits_equal(a_buf, want_ag, "all-gather input with its guard lanes")
    pos = 0
    for i, n in enumerate(numels):
        ref = torch.full((n + offs[i] + 9,), 3.0, dtype=param_dt)
        if modes[i]:
            ref[offs[i] : offs[i] + n].copy_(gathered[pos : pos + n])
        assert_bits_equal(bufs[i], ref, f"tensor {i} with its guard lanes")
        pos += n
    table.close()


@settings(max_examples=100 * SCALE, **COMMON)
@given(numels=tables, pad=st.integers(0, 700), grad_dt=st.sampled_from(DTYPES), wide_buffer=st.booleans(),
       shard_dt=st.sampled_from(DTYPES), acc=st.booleans(), two_waves=st.booleans(), zero_pad=st.booleans(),
       seed=st.integers(0, 2**20), policy=policies)
def test_gather_in_post_reduce_any_table(nat, numels, pad, grad_dt, wide_buffer, shard_dt, acc, two_waves, zero_pad, seed, policy):
    nat.set_store_policy(policy)
    """Reduce copy-in and post-reduce of a size-one group as one launch: the reduce buffer (guard lanes included)
    and the gradient shard against the reference's op sequence."""
    rs_dt = torch.float32 if wide_buffer else grad_dt
    print("gather_in_post_reduce", numels, pad, grad_dt, rs_dt, shard_dt, acc, two_waves, zero_pad, seed, flush=True)
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    p, t = len(numels), sum(numels)
    t_pad = t + pad
    grads = [mixed_values(g, n, grad_dt, 1e-3) for n in numels]
    modes = rng.integers(0, 3, size=p).tolist()
    old = torch.zeros(t_pad + 8, dtype=rs_dt)
    old[:t_pad] = mixed_values(g, t_pad, rs_dt, 1e-3).flip(0)
    old[t_pad:] = 5.0
    shard0 = mixed_values(g, t_pad, shard_dt, 1e-3, specials=False)
    want = old.clone()
    views = list(want[:t].split(numels))
    cp = [i for i, m in enumerate(modes) if m == 1]
    ad = [i for i, m in enumerate(modes) if m == 2]
    torch_ops.reduce_copy_in([views[i] for i in cp], [grads[i] for i in cp], False)
    torch_ops.reduce_copy_in([views[i] for i in ad], [grads[i] for i in ad], True)
    if zero_pad:
        want[t:t_pad] = 0
    want_shard = shard0.clone()
    torch_ops.reduce_scatter_local(want_shard, want[:t_pad].clone(), 1, 0, None, None, "add" if acc else "copy")
    default = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_TABLE_LARGE_LOG2, 0 if two_waves else default)
    try:
        table = nat.TensorTable(numels, t_pad, DEV)
    finally:
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default)
    got, got_shard = old.to(DEV), shard0.to(DEV)
    dgrads = [_view_at(x, int(rng.integers(0, 8)))[1] for x in grads]
    assert table.gather_in_post_reduce(dgrads, got, got_shard, acc, modes, zero_pad=zero_pad)
    assert_bits_equal(got, want, "reduce buffer")
    assert_bits_equal(got_shard, want_shard, "gradient shard")
    table.close()


# ------------------------------------------------------------ optimizer side --
@settings(max_examples=80 * SCALE, **COMMON)
@given(n=st.integers(1, 40_000), off=st.integers(0, 3), decoupled=st.booleans(),
       beta1=st.sampled_from([0.9, 0.5, 0.3, 0.0]), beta2=st.sampled_from([0.95, 0.999, 0.5]),
       wd=st.sampled_from([0.0, 0.1, 1e-2]), lr=st.sampled_from([3e-4, 1e-2, 0.0]), step=st.integers(1, 2000),
       out_dt=st.sampled_from([None, torch.bfloat16, torch.float16]), gscale=st.sampled_from([None, 0.5, 0.19153, 1.0]),
       zero_grad=st.booleans(), seed=st.integers(0, 2**20), policy=policies)
def test_adamw_any_shape(nat, n, off, decoupled, beta1, beta2, wd, lr, step, out_dt, gscale, zero_grad, seed, policy):
    nat.set_store_policy(policy)
    from oracle import cref

    print("adamw", n, off, decoupled, beta1, beta2, wd, lr, step, out_dt, gscale, zero_grad, seed, flush=True)
    g = torch.Generator().manual_seed(seed)
    hp = dict(lr=lr, beta1=beta1, beta2=beta2, eps=1e-8, weight_decay=wd)
    p = mixed_values(g, n, torch.float32, 0.02)
    grad = mixed_values(g, n, torch.float32, 1e-3).flip(0).contiguous()
    m = mixed_values(g, n, torch.float32, 1e-3, specials=False)
    v = mixed_values(g, n, torch.float32, 1e-3, specials=False) ** 2
    full = [torch.full((n + 8,), 5.0, device=DEV) for _ in range(4)]
    dev = [f[off : off + n].copy_(t) for f, t in zip(full, (p, grad, m, v))]
    out = None if out_dt is None else torch.full((n + 8,), 9.0, dtype=out_dt, device=DEV)
    gs = None if gscale is None else torch.tensor([gscale], device=DEV)
    nat.adamw_step(dev[0], dev[1], dev[2], dev[3], None if out is None else out[off : off + n], step=step,
                   decoupled=decoupled, grad_scale=gs, zero_grad=zero_grad, **hp)
    want_out = None if out_dt is None else torch.full((n + 8,), 9.0, dtype=out_dt)
    cref.adamw_step(p, grad, m, v, None if want_out is None else want_out[off : off + n], step=step,
                    decoupled=decoupled, grad_scale=gscale, zero_grad=zero_grad, **hp)
    for name, f, b in zip(("param", "grad", "exp_avg", "exp_avg_sq"), full, (p, grad, m, v)):
        want_full = torch.full((n + 8,), 5.0)
        want_full[off : off + n] = b
        assert_bits_equal(f, want_full, name)
    if out is not None:
        assert_bits_equal(out, want_out, "out16")


@settings(max_examples=60 * SCALE, **COMMON)
@given(dt=st.sampled_from(DTYPES), n=st.integers(0, 300_000), off=st.integers(0, 8),
       coef=st.sampled_from([1.0, 0.5, 0.19153, 3.0]), seed=st.integers(0, 2**20), policy=policies)
def test_sumsq_fill_scale_any_shape(nat, dt, n, off, coef, seed, policy):
    nat.set_store_policy(policy)
    import math

    from oracle import cref

    print("sumsq/scale/fill", dt, n, off, coef, seed, flush=True)
    g = torch.Generator().manual_seed(seed)
    x = mixed_values(g, n, dt, 3e-2, specials=False)
    buf, d = _view_at(x, off, fill=7.0)
    ws = nat.sumsq_workspace(DEV)
    out = torch.zeros(1, dtype=torch.float64, device=DEV)
    nat.flat_sumsq(d, out, ws, accumulate=False)
    want = cref.sumsq(x)
    assert math.isclose(float(out), want, rel_tol=1e-12, abs_tol=1e-300), (float(out), want)
    nat.flat_scale(d, torch.tensor([coef], device=DEV))
    ref = x.clone()
    cref.flat_scale(ref, coef)
    assert_bits_equal(d, ref, "scale")
    nat.flat_fill(d, -0.25)
    assert int((d.float() != -0.25).sum()) == 0
    guard = torch.cat([buf[:off], buf[off + n :]]).float()
    assert float(guard.min()) == 7.0 and float(guard.max()) == 7.0


@settings(max_examples=60 * SCALE, **COMMON)
@given(src_dt=st.sampled_from(DTYPES), dst_dt=st.sampled_from(DTYPES), n=st.integers(0, 60_000),
       k=st.integers(1, 16), seed=st.integers(0, 2**20), policy=policies)
def test_fanout_any_shape(nat, src_dt, dst_dt, n, k, seed, policy):
    nat.set_store_policy(policy)
    print("fanout", src_dt, dst_dt, n, k, seed, flush=True)
    g = torch.Generator().manual_seed(seed)
    src = mixed_values(g, n, src_dt)
    want = torch.empty(n, dtype=dst_dt)
    torch_ops.copy_in(want, src)
    dsts = [torch.full((n,), 3.0, dtype=dst_dt, device=DEV) for _ in range(k)]
    nat.flat_copy_fanout(dsts, src.to(DEV))
    for i, d in enumerate(dsts):
        assert_bits_equal(d, want, f"destination {i}")


@settings(max_examples=60 * SCALE, **COMMON)
@given(chunk_dt=st.sampled_from(DTYPES), shard_dt=st.sampled_from(DTYPES), n=st.integers(0, 60_000),
       k=st.integers(1, 16), post=st.sampled_from(FACTORS), acc=st.booleans(), seed=st.integers(0, 2**20), policy=policies)
def test_fanin_any_shape(nat, chunk_dt, shard_dt, n, k, post, acc, seed, policy):
    nat.set_store_policy(policy)
    print("fanin", chunk_dt, shard_dt, n, k, post, acc, seed, flush=True)
    g = torch.Generator().manual_seed(seed)
    chunks = [mixed_values(g, n, chunk_dt, 1e-3).roll(i) for i in range(k)]
    shard0 = mixed_values(g, n, shard_dt, 1e-4).flip(0).contiguous()
    want = shard0.clone()
    torch_ops.reduce_scatter_fanin(want, [c.clone() for c in chunks], post, acc)
    got = shard0.to(DEV)
    nat.post_reduce_fanin(got, [c.to(DEV) for c in chunks], post, acc)
    assert_bits_equal(got, want, "shard")


# ------------------------------------------------------------- group level --
shape_st = st.one_of(st.tuples(st.integers(1, 300)), st.tuples(st.integers(1, 40), st.integers(1, 40)),
                     st.tuples(st.integers(1, 6), st.integers(1, 9), st.integers(1, 9)))


@settings(max_examples=40 * SCALE, **COMMON)
@given(shapes=st.lists(shape_st, min_size=1, max_size=6), w=st.integers(1, 6), r_frac=st.floats(0, 0.999),
       align=st.sampled_from([1, 2, 8, 16]), policy=st.sampled_from(["bf16", "bf16-fp32reduce", "fp16"]),
       iterations=st.integers(1, 3), seed=st.integers(0, 2**20))
def test_param_group_any_layout(shapes, w, r_frac, align, policy, iterations, seed):
    """A parameter group with drawn shapes, world size, rank, alignment and precision policy through
    unshard -> backward -> reduce for a few iterations (some parameters without a gradient in some of them),
    against the reference's op sequence on CPU tensors."""
    from test_gpu_param_group import CpuGroup, _make_group, _run_backward

    from yafsdp_amd import MixedPrecisionPolicy

    r = int(r_frac * w)
    print("param group", shapes, w, r, align, policy, iterations, seed, flush=True)
    low = torch.float16 if policy == "fp16" else torch.bfloat16
    mp = MixedPrecisionPolicy(param_dtype=low, reduce_dtype=torch.float32 if policy == "bf16-fp32reduce" else None)
    if policy == "fp16":  # ya_fsdp/_collectives.py:252-262
        pre = 1
        while w % pre == 0 and w / pre > pre:
            pre *= 2
        pre, post = float(pre), float(w / pre)
        collective = None
    else:                 # AVG inside the collective: this rank's share is its chunk times 1 / W rounded to the dtype
        pre, post = None, None
        collective = ("AVG", None) if w > 1 else None
    group, cpu_params = _make_group(shapes, w, r, align, mp, seed=seed % 1000)
    ref = CpuGroup(cpu_params, w, r, align, mp)
    rng = np.random.default_rng(seed)
    owns = [False] * len(shapes)  # parameters whose sharded gradient exists already
    for it in range(iterations):
        group.pre_forward(); group.post_forward(); group.pre_backward()
        got_views = [fp.unsharded_param for fp in group.fsdp_params]
        for v, w_ in zip(got_views, ref.unshard(first_of_iteration=True)):
            assert_bits_equal(v.detach(), w_, "unsharded parameter")
        g = torch.Generator().manual_seed(seed + it)
        grads = [(torch.randn(s, generator=g) * 1e-3).to(low) for s in shapes]
        present = rng.random(len(shapes)) < 0.8
        if not present.any():
            present[int(rng.integers(0, len(shapes)))] = True
        grads = [x if p else None for x, p in zip(grads, present)]
        _run_backward(group, ref, grads)
        with_grad = [i for i, x in enumerate(grads) if x is not None]
        if all(not owns[i] for i in with_grad) and len(with_grad) == len(shapes):
            ref.reduce(pre, post, "copy", collective=collective)
        elif all(owns[i] for i in with_grad) and len(with_grad) == len(shapes):
            ref.reduce(pre, post, "add", collective=collective)
        else:
            ref.reduce(pre, post, "mixed", [None if x is None else owns[i] for i, x in enumerate(grads)],
                       collective=collective)
        for i in with_grad:
            owns[i] = True
        group.finalize_backward()
        torch.cuda.synchronize()
        got, want = group._padded_sharded_param_grad[None], ref.grad_shard
        # fragments of parameters that never had a gradient hold unspecified values in the reference; compare the
        # fragments that are defined
        pos = 0
        for i, n in enumerate(ref.lay.sharded_numels(r)):
            if owns[i]:
                assert_bits_equal(got[pos : pos + n], want[pos : pos + n], f"gradient fragment {i}, iteration {it}")
            pos += n


@settings(max_examples=30 * SCALE, **COMMON)
@given(spec=st.lists(st.tuples(shape_st, st.booleans()), min_size=1, max_size=7), w=st.integers(1, 5),
       r_frac=st.floats(0, 0.999), align=st.sampled_from([1, 2, 8, 16]), iterations=st.integers(1, 3),
       seed=st.integers(0, 2**20))
def test_param_group_with_all_gather_dtype_classes(spec, w, r_frac, align, iterations, seed):
    """A group whose parameters are split at random between the default class and a tensor-subclass class with an
    int8 all-gather (ya_fsdp/_param_group.py:194-227): per class the all-gather input, this rank's slot of the
    gathered buffer and the gradient shard over a few iterations with missing gradients, against the reference's op
    sequence on CPU tensors."""
    import torch.nn as nn
    from ext_subclasses import Int8Master, quantize
    from test_gpu_param_group import BF16_MP, CpuGroup

    from yafsdp_amd import FSDPMeshInfo, MixedPrecisionPolicy
    from yafsdp_amd._param_group import YaFSDPParamGroup, init_shared_state

    r = int(r_frac * w)
    print("classes", spec, w, r, align, iterations, seed, flush=True)
    g = torch.Generator().manual_seed(seed)
    values = [torch.randn(s, generator=g) * 0.08 for s, _ in spec]
    dev_params = [nn.Parameter(Int8Master(v.to(DEV))) if ext else v.to(DEV).requires_grad_(True)
                  for v, (_, ext) in zip(values, spec)]
    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16, all_gather_dtype_to_param_cls={torch.int8: Int8Master})
    group = YaFSDPParamGroup(dev_params, FSDPMeshInfo(w, r), DEV, mp, align)
    init_shared_state([group], DEV)
    keys = {None: [i for i, (_, e) in enumerate(spec) if not e], torch.int8: [i for i, (_, e) in enumerate(spec) if e]}
    keys = {k: idx for k, idx in keys.items() if idx}
    assert list(group._all_gather_dtype_to_fsdp_params) == list(keys)
    refs = {k: CpuGroup([values[i] for i in idx], w, r, align, BF16_MP) for k, idx in keys.items()}
    collective = ("AVG", None) if w > 1 else None  # bf16 reduce: the collective scales by 1 / W rounded to bf16
    rng = np.random.default_rng(seed)
    owns = [False] * len(spec)
    for it in range(iterations):
        group.pre_forward(); group.post_forward(); group.pre_backward()
        torch.cuda.synchronize()
        for k, ref in refs.items():
            n_local = ref.lay.sharded_numels(r)
            if k is None:
                torch_ops.copy_in(ref.ag_in, ref.shard)
                want_in = ref.ag_in
            else:
                want_in = torch.zeros(ref.lay.padded_sharded_numel, dtype=torch.int8)
                for dst, frag in zip(want_in[: sum(n_local)].split(n_local), ref.shard[: sum(n_local)].split(n_local)):
                    torch_ops.extension_copy_in(dst, quantize(frag))
            got_in, got_out = group._all_gather_input[k].cpu(), group._all_gather_output[k].cpu()
            s_ = ref.lay.padded_sharded_numel
            assert torch.equal(got_in.view(torch.uint8), want_in.view(torch.uint8)), (k, "all-gather input")
            assert torch.equal(got_out[r * s_ : (r + 1) * s_].view(torch.uint8), got_in.view(torch.uint8)), (k, "slot")
        gg = torch.Generator().manual_seed(seed + 1 + it)
        grads = [(torch.randn(s, generator=gg) * 1e-3).bfloat16() for s, _ in spec]
        present = rng.random(len(spec)) < 0.8
        if not present.any():
            present[int(rng.integers(0, len(spec)))] = True
        grads = [x if p else None for x, p in zip(grads, present)]
        for fp, x in zip(group.fsdp_params, grads):
            fp.unsharded_param.grad = None if x is None else x.to(DEV)
        group.post_backward()
        group.finalize_backward()
        torch.cuda.synchronize()
        for k, ref in refs.items():
            mine = [grads[i] for i in keys[k]]
            mine_owns = [owns[i] for i in keys[k]]
            if all(x is None for x in mine):
                continue  # the class took no part in this pass: its gradient shard is untouched
            ref.accumulate(mine, [False] * len(mine))
            with_grad = [j for j, x in enumerate(mine) if x is not None]
            if all(not mine_owns[j] for j in with_grad) and len(with_grad) == len(mine):
                ref.reduce(None, None, "copy", collective=collective)
            elif all(mine_owns[j] for j in with_grad) and len(with_grad) == len(mine):
                ref.reduce(None, None, "add", collective=collective)
            else:
                ref.reduce(None, None, "mixed", [None if x is None else mine_owns[j] for j, x in enumerate(mine)],
                           collective=collective)
        for i, x in enumerate(grads):
            if x is not None:
                owns[i] = True
        for k, ref in refs.items():
            got, want = group._padded_sharded_param_grad[k], ref.grad_shard
            pos = 0
            for j, n in enumerate(ref.lay.sharded_numels(r)):
                if owns[keys[k][j]]:
                    assert_bits_equal(got[pos : pos + n], want[pos : pos + n], f"class {k} fragment {j}, iteration {it}")
                pos += n
