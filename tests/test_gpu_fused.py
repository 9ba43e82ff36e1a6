"""GPU parity of the two launches that do the work of two each, through the C ABI: against the oracle's torch ops
(the reference's own calls) and against the separate entry points they stand for."""

from __future__ import annotations

import sys

import numpy as np
import pytest
import torch

from oracle import torch_ops
from tests.helpers import DTYPES, assert_bits_equal, mixed_values

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def nat():
    from yafsdp_amd import _native

    return _native


def _say(*a):
    print(*a, file=sys.stderr, flush=True)


def _numels(rng, p, max_log2, with_empty):
    n = np.floor(np.exp2(rng.uniform(0, max_log2, size=p))).astype(np.int64) | 1
    if with_empty and p > 3:
        n[rng.integers(0, p, size=max(1, p // 10))] = 0
    return n.tolist()


# (P, max log2 numel, with_empty, pad, line_aligned)
CASES = [
    (1, 3, False, 0, False),
    (3, 4, False, 5, False),
    (9, 16, True, 17, False),
    (16, 14, True, 9, False),
    (9, 17, False, 64, True),
    (7, 19, False, 513, False),
    (33, 14, True, 9, False),      # more than 16 tensors: records and per-call pointers in device memory
    (200, 12, True, 4096, False),
    (40, 12, False, 0, True),
]


def _case_numels(case, salt):
    p, max_log2, with_empty, pad, aligned = case
    rng = np.random.default_rng(p * 1000 + pad + salt)
    numels = _numels(rng, p, max_log2, with_empty)
    if aligned:  # every tensor starts on a 128-byte line of a bf16 buffer: the short scatter-out tile
        numels = [((n + 63) // 64) * 64 for n in numels]
    return rng, numels


# ----------------------------------------------------- copy-in + copy-out --
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("master_dt,param_dt", [(torch.float32, torch.bfloat16), (torch.float32, torch.float16),
                                                (torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                                (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("shard_n", [0, 1, 77, 4099, 300_001])
def test_copy_in_scatter_out(nat, case, master_dt, param_dt, shard_n):
    rng, numels = _case_numels(case, 11)
    pad = case[3]
    t = sum(numels)
    g = torch.Generator().manual_seed(301 + case[0] + shard_n % 7)
    _say("copy_in_scatter_out", case, master_dt, param_dt, shard_n, "T", t)
    gathered = mixed_values(g, t + pad, param_dt)
    master = mixed_values(g, shard_n + 3, master_dt)
    # oracle: the cast of the master shard and the split of the gathered buffer
    want_ag = torch.full((shard_n + 5,), 3.0, dtype=param_dt)
    torch_ops.copy_in(want_ag[1 : 1 + shard_n], master[3:])
    want = [torch.full((n + 2,), 3.0, dtype=param_dt) for n in numels]
    torch_ops.copy_out_materialize(gathered, numels, [w[1 : 1 + n] for w, n in zip(want, numels)])
    table = nat.TensorTable(numels, t + pad, torch.device(DEV))
    got_ag = torch.full((shard_n + 5,), 3.0, dtype=param_dt, device=DEV)
    got = [torch.full((n + 2,), 3.0, dtype=param_dt, device=DEV) for n in numels]
    dmaster, dgathered = master.to(DEV), gathered.to(DEV)
    served = table.copy_in_scatter_out(
        dgathered, [x[1 : 1 + n] for x, n in zip(got, numels)], got_ag[1 : 1 + shard_n], dmaster[3:]
    )
    assert served
    assert_bits_equal(got_ag, want_ag, "all-gather input (guard lanes included)")
    for i, (a, b) in enumerate(zip(got, want)):
        assert_bits_equal(a, b, f"tensor {i}")
    # the separate entry points give the same bytes
    two_ag = torch.full((shard_n + 5,), 3.0, dtype=param_dt, device=DEV)
    two = [torch.full((n + 2,), 3.0, dtype=param_dt, device=DEV) for n in numels]
    nat.flat_copy(two_ag[1 : 1 + shard_n], dmaster[3:])
    table.scatter_out(dgathered, [x[1 : 1 + n] for x, n in zip(two, numels)])
    assert torch.equal(two_ag.view(torch.uint8), got_ag.view(torch.uint8))
    for a, b in zip(two, got):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    # skip modes leave their tensors alone
    if len(numels) > 1:
        modes = rng.integers(0, 2, size=len(numels)).tolist()
        got2 = [torch.full((n,), 3.0, dtype=param_dt, device=DEV) for n in numels]
        got_ag.fill_(3.0)
        assert table.copy_in_scatter_out(dgathered, got2, got_ag[1 : 1 + shard_n], dmaster[3:], modes)
        assert_bits_equal(got_ag, want_ag, "all-gather input, call with modes")
        pos = 0
        for i, n in enumerate(numels):
            ref = torch.full((n,), 3.0, dtype=param_dt)
            if modes[i]:
                ref.copy_(gathered[pos : pos + n])
            assert_bits_equal(got2[i], ref, f"modes tensor {i}")
            pos += n
    table.close()


@pytest.mark.parametrize("tail_mb", [0, 1, 3])
@pytest.mark.parametrize("two_waves", [False, True])
@pytest.mark.parametrize("master_dt,param_dt", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_copy_out_with_the_write_through_boundary_inside_the_tensors(nat, tail_mb, two_waves, master_dt, param_dt):
    """The tile slots of the last megabytes of tensors are stored with another cache policy than the rest (0: none
    are; the default is larger than all tensors of the other tests together, so there all are), in the shared launch
    and in scatter-out as a launch of its own.  Same bytes either way."""
    default_tail = nat.get_option(nat.OPT_SCATTER_TAIL_MB)
    default_flat_tail = nat.get_option(nat.OPT_FLAT_TAIL_MB)
    default_log2 = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_SCATTER_TAIL_MB, tail_mb)
    nat.set_option(nat.OPT_FLAT_TAIL_MB, tail_mb)  # the cast part of the shared launch: the same kind of boundary
    if two_waves:
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, 0)
    try:
        for case, shard_n in [((7, 19, False, 513, False), 1_300_001), ((9, 17, False, 64, True), 4099),
                              ((33, 14, True, 9, False), 4099), ((5, 21, False, 0, True), 2_000_003)]:
            test_copy_in_scatter_out(nat, case, master_dt, param_dt, shard_n)
    finally:
        nat.set_option(nat.OPT_SCATTER_TAIL_MB, default_tail)
        nat.set_option(nat.OPT_FLAT_TAIL_MB, default_flat_tail)
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default_log2)


def test_copy_in_scatter_out_declines_and_errors(nat):
    flat = torch.ones(16, dtype=torch.bfloat16, device=DEV)
    ag = torch.zeros(8, dtype=torch.bfloat16, device=DEV)
    master = torch.ones(8, dtype=torch.float32, device=DEV)
    table = nat.TensorTable([8, 8], 16, torch.device(DEV))
    outs = [torch.zeros(8, dtype=torch.float32, device=DEV) for _ in range(2)]
    assert table.copy_in_scatter_out(flat, outs, ag, master) is False  # tensors of another dtype than the buffer
    torch.cuda.synchronize()
    assert float(ag.float().abs().sum()) == 0.0 and all(float(o.abs().sum()) == 0.0 for o in outs)
    with pytest.raises(ValueError):
        table.copy_in_scatter_out(flat, [o.bfloat16() for o in outs], ag[:4], master)
    with pytest.raises(RuntimeError):  # in-place cast
        both = torch.zeros(16, dtype=torch.float32, device=DEV)
        table.copy_in_scatter_out(flat, [o.bfloat16() for o in outs], both.view(torch.bfloat16)[:8], both[:8])
    table.close()


@pytest.mark.parametrize("two_waves", [False, True])
def test_both_launches_at_both_workgroup_sizes(nat, two_waves):
    """Tables above the size threshold run two waves per workgroup (gather-in side always, scatter-out side unless
    every tensor starts on a cache line): the shared launches follow the table."""
    default = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_TABLE_LARGE_LOG2, 0 if two_waves else default)
    try:
        for p in (5, 40):
            rng = np.random.default_rng(70 + p)
            numels = _numels(rng, p, 13, True)
            t, pad = sum(numels), 24
            g = torch.Generator().manual_seed(71 + p)
            gathered = mixed_values(g, t + pad, torch.bfloat16)
            master = mixed_values(g, 5000, torch.float32)
            grads = [mixed_values(g, n, torch.bfloat16, 1e-3) for n in numels]
            old = mixed_values(g, t + pad, torch.bfloat16, 1e-3)
            shard0 = mixed_values(g, t + pad, torch.float32, 1e-3, specials=False)
            table = nat.TensorTable(numels, t + pad, torch.device(DEV))
            got = [torch.full((n,), 3.0, dtype=torch.bfloat16, device=DEV) for n in numels]
            ag = torch.zeros(5000, dtype=torch.bfloat16, device=DEV)
            assert table.copy_in_scatter_out(gathered.to(DEV), got, ag, master.to(DEV))
            want_ag = torch.zeros(5000, dtype=torch.bfloat16)
            torch_ops.copy_in(want_ag, master)
            assert_bits_equal(ag, want_ag, "all-gather input")
            want = [torch.empty(n, dtype=torch.bfloat16) for n in numels]
            torch_ops.copy_out_materialize(gathered, numels, want)
            for i, (a, b) in enumerate(zip(got, want)):
                assert_bits_equal(a, b, f"tensor {i}")
            want_flat = old.clone()
            torch_ops.reduce_copy_in(list(want_flat[:t].split(numels)), grads, False)
            want_flat[t:].zero_()
            want_shard = shard0.clone()
            torch_ops.reduce_scatter_local(want_shard, want_flat.clone(), 1, 0, None, None, "add")
            got_flat, got_shard = old.to(DEV), shard0.to(DEV)
            assert table.gather_in_post_reduce([x.to(DEV) for x in grads], got_flat, got_shard, True)
            assert_bits_equal(got_flat, want_flat, "reduce buffer")
            assert_bits_equal(got_shard, want_shard, "gradient shard")
            table.close()
    finally:
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default)


# --------------------------------------------- reduce copy-in + post-reduce --
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("grad_dt,rs_dt,shard_dt", [
    (torch.bfloat16, torch.bfloat16, torch.float32),
    (torch.bfloat16, torch.float32, torch.float32),
    (torch.float32, torch.float32, torch.float32),
    (torch.float16, torch.float16, torch.float32),
    (torch.bfloat16, torch.bfloat16, torch.bfloat16),
    (torch.float16, torch.float32, torch.float16),
])
@pytest.mark.parametrize("acc", [False, True])
@pytest.mark.parametrize("zero_pad", [True, False])
def test_gather_in_post_reduce(nat, case, grad_dt, rs_dt, shard_dt, acc, zero_pad):
    rng, numels = _case_numels(case, 12)
    p, pad = len(numels), case[3]
    t = sum(numels)
    t_pad = t + pad
    g = torch.Generator().manual_seed(311 + p)
    _say("gather_in_post_reduce", case, grad_dt, rs_dt, shard_dt, acc, zero_pad, "T", t)
    grads = [mixed_values(g, n, grad_dt, 1e-3) for n in numels]
    modes = rng.integers(0, 3, size=p).tolist() if p > 1 else [1]
    old = torch.zeros(t_pad + 8, dtype=rs_dt)
    old[:t_pad] = mixed_values(g, t_pad, rs_dt, 1e-3).flip(0)
    old[t_pad:] = 5.0
    shard0 = mixed_values(g, t_pad, shard_dt, 1e-3, specials=False)
    # oracle: foreach copy / foreach add into the views of the reduce buffer, pad zeroed, then the shard group of
    # size one's "reduce-scatter" (the buffer itself) copied or added into the gradient shard
    want_flat = old.clone()
    views = list(want_flat[:t].split(numels))
    cp = [i for i, m in enumerate(modes) if m == 1]
    ad = [i for i, m in enumerate(modes) if m == 2]
    torch_ops.reduce_copy_in([views[i] for i in cp], [grads[i] for i in cp], False)
    torch_ops.reduce_copy_in([views[i] for i in ad], [grads[i] for i in ad], True)
    if zero_pad:
        want_flat[t:t_pad].zero_()
    want_shard = shard0.clone()
    torch_ops.reduce_scatter_local(want_shard, want_flat[:t_pad].clone(), 1, 0, None, None, "add" if acc else "copy")
    table = nat.TensorTable(numels, t_pad, torch.device(DEV))
    got_flat, got_shard = old.to(DEV), shard0.to(DEV)
    dgrads = [torch.cat([x.new_zeros(i % 5), x]).to(DEV)[i % 5 :] for i, x in enumerate(grads)]
    assert table.gather_in_post_reduce(dgrads, got_flat, got_shard, acc, modes, zero_pad=zero_pad)
    assert_bits_equal(got_flat, want_flat, "reduce buffer afterwards (guard lanes included)")
    assert_bits_equal(got_shard, want_shard, "gradient shard")
    # the two separate calls give the same bytes
    two_flat, two_shard = old.to(DEV), shard0.to(DEV)
    table.gather_in(dgrads, two_flat, modes, None, zero_pad=zero_pad)
    nat.post_reduce(two_shard, two_flat[:t_pad], None, acc)
    assert_bits_equal(got_flat, two_flat, "reduce buffer against the two calls")
    assert_bits_equal(got_shard, two_shard, "gradient shard against the two calls")
    table.close()


@pytest.mark.parametrize("case", [CASES[2], CASES[4], CASES[6]])
@pytest.mark.parametrize("grad_dt,rs_dt,shard_dt", [
    (torch.bfloat16, torch.bfloat16, torch.float32),
    (torch.float16, torch.float16, torch.float32),
    (torch.bfloat16, torch.float32, torch.bfloat16),
])
@pytest.mark.parametrize("factors", [
    # (pre, custom, post)
    (None, None, 8.0), (None, None, 3.0), (4.0, None, 2.0), (16.0, None, 16.0), (3.0, None, None),
    (None, 4.0, None), (None, 3.0, None), (None, 0.5, None), (None, -7.0, None), (None, 1.0, None), (1.0, None, 0.5),
])
@pytest.mark.parametrize("acc", [False, True])
def test_gather_in_post_reduce_with_divide_factors(nat, case, grad_dt, rs_dt, shard_dt, factors, acc):
    """The divides of the reduce step inside the one-pass reduce: the pre-divide and the custom division act on the
    reduce buffer in place (ya_fsdp/_collectives.py:139, 146-148), the post-divide on what goes on to the shard
    (:165); each rounds to the buffer's dtype.  Against the op sequence and against the separate entry points."""
    pre, custom, post = factors
    rng, numels = _case_numels(case, 13)
    p, pad = len(numels), case[3]
    t = sum(numels)
    t_pad = t + pad
    g = torch.Generator().manual_seed(331 + p)
    _say("gather_in_post_reduce factors", case, grad_dt, rs_dt, shard_dt, factors, acc)
    grads = [mixed_values(g, n, grad_dt, 1e-3) for n in numels]
    modes = rng.integers(0, 3, size=p).tolist()
    old = mixed_values(g, t_pad, rs_dt, 1e-3).flip(0).contiguous()
    shard0 = mixed_values(g, t_pad, shard_dt, 1e-3, specials=False)
    want_flat = old.clone()
    views = list(want_flat[:t].split(numels))
    cp = [i for i, m in enumerate(modes) if m == 1]
    ad = [i for i, m in enumerate(modes) if m == 2]
    torch_ops.reduce_copy_in([views[i] for i in cp], [grads[i] for i in cp], False)
    torch_ops.reduce_copy_in([views[i] for i in ad], [grads[i] for i in ad], True)
    want_flat[t:].zero_()
    torch_ops.div_if_needed(want_flat, pre)                      # :139
    if custom is not None:
        want_flat.copy_(want_flat / custom)                      # :146-148 (output aliases the input at size one)
    want_shard = shard0.clone()
    torch_ops.reduce_scatter_local(want_shard, want_flat.clone(), 1, 0, None, post, "add" if acc else "copy")
    table = nat.TensorTable(numels, t_pad, torch.device(DEV))
    dgrads = [x.to(DEV) for x in grads]
    got_flat, got_shard = old.to(DEV), shard0.to(DEV)
    assert table.gather_in_post_reduce(dgrads, got_flat, got_shard, acc, modes, pre_factor=pre, post_factor=post,
                                       custom_divisor=custom)
    assert_bits_equal(got_flat, want_flat, "reduce buffer (before the post-divide)")
    assert_bits_equal(got_shard, want_shard, "gradient shard")
    two_flat, two_shard = old.to(DEV), shard0.to(DEV)
    table.gather_in(dgrads, two_flat, modes, pre, zero_pad=True)
    if custom is not None:
        nat.flat_div_copy(two_flat, two_flat, custom)
    nat.post_reduce(two_shard, two_flat, post, acc)
    assert_bits_equal(got_flat, two_flat, "reduce buffer against the separate calls")
    assert_bits_equal(got_shard, two_shard, "gradient shard against the separate calls")
    table.close()


def test_gather_in_post_reduce_declines_and_errors(nat):
    grads = [torch.ones(40, dtype=torch.bfloat16, device=DEV) for _ in range(2)]
    flat = torch.zeros(96, dtype=torch.bfloat16, device=DEV)
    shard = torch.zeros(96, dtype=torch.float32, device=DEV)
    table = nat.TensorTable([40, 40], 96, torch.device(DEV))
    # float32 gradients into a bf16 reduce buffer: not in the list of the fused launch
    assert table.gather_in_post_reduce([g.float() for g in grads], flat, shard, False) is False
    torch.cuda.synchronize()
    assert float(shard.abs().sum()) == 0.0 and float(flat.float().abs().sum()) == 0.0
    with pytest.raises(ValueError):
        table.gather_in_post_reduce(grads, flat, shard[:95], False)
    with pytest.raises(RuntimeError):  # shard not 16-byte aligned
        wide = torch.zeros(97, dtype=torch.float32, device=DEV)
        table.gather_in_post_reduce(grads, flat, wide[1:], False)
    with pytest.raises(RuntimeError):  # shard inside the reduce buffer
        both = torch.zeros(96, dtype=torch.float32, device=DEV)
        table.gather_in_post_reduce([g.float() for g in grads], both, both, False)
    with pytest.raises(RuntimeError):  # the custom division excludes the other two factors
        table.gather_in_post_reduce(grads, flat, shard, False, pre_factor=2.0, custom_divisor=3.0)
    with pytest.raises(RuntimeError):
        table.gather_in_post_reduce(grads, flat, shard, False, custom_divisor=float("inf"))
    table.close()


def test_changing_pointer_sets_on_a_large_table(nat):
    """A table with more than 16 tensors stages its per-call pointers: unchanged and changed sets alternate, every
    call against the oracle."""
    rng = np.random.default_rng(81)
    numels = _numels(rng, 60, 10, True)
    t = sum(numels)
    g = torch.Generator().manual_seed(82)
    table = nat.TensorTable(numels, t + 16, torch.device(DEV))
    shard_cpu = torch.zeros(t + 16, dtype=torch.float32)
    shard = shard_cpu.to(DEV)
    flat = torch.zeros(t + 16, dtype=torch.bfloat16, device=DEV)
    flat_cpu = torch.zeros(t + 16, dtype=torch.bfloat16)
    sets = [[mixed_values(g, n, torch.bfloat16, 1e-3, specials=False) for n in numels] for _ in range(3)]
    dsets = [[x.to(DEV) for x in s_] for s_ in sets]
    for k in (0, 0, 1, 0, 2, 2, 1):
        assert table.gather_in_post_reduce(dsets[k], flat, shard, True)
        torch_ops.reduce_copy_in(list(flat_cpu[:t].split(numels)), sets[k], False)
        torch_ops.reduce_scatter_local(shard_cpu, flat_cpu.clone(), 1, 0, None, None, "add")
        assert_bits_equal(shard, shard_cpu, f"gradient shard after set {k}")
    table.close()


@pytest.mark.parametrize("dt", DTYPES)
def test_gather_in_post_reduce_empty_table(nat, dt):
    table = nat.TensorTable([], 0, torch.device(DEV))
    flat = torch.zeros(0, dtype=dt, device=DEV)
    shard = torch.zeros(0, dtype=torch.float32, device=DEV)
    assert table.gather_in_post_reduce([], flat, shard, True)
    table.close()
