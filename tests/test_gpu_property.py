"""Randomised parity of the buffer-path kernels against the oracle (hypothesis, derandomised: the same
examples on every run).  Shapes, dtypes, alignments, factors and per-tensor modes are drawn together, which
reaches combinations the parametrised tests do not enumerate.  Each example is small; every one names itself
on stdout before it touches the GPU."""

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
COMMON = dict(deadline=None, derandomize=True, suppress_health_check=list(HealthCheck), print_blob=False)


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


@settings(max_examples=120, **COMMON)
@given(src_dt=st.sampled_from(DTYPES), dst_dt=st.sampled_from(DTYPES), n=st.integers(0, 70_000),
       s_off=st.integers(0, 8), d_off=st.integers(0, 8), factor=st.sampled_from(FACTORS), acc=st.booleans(),
       seed=st.integers(0, 2**20))
def test_post_reduce_any_shape(nat, src_dt, dst_dt, n, s_off, d_off, factor, acc, seed):
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


tables = st.lists(st.one_of(st.just(0), st.integers(1, 40), st.integers(1, 6000)), min_size=1, max_size=40)


@settings(max_examples=80, **COMMON)
@given(numels=tables, pad=st.integers(0, 700), grad_dt=st.sampled_from(DTYPES), rs_dt=st.sampled_from(DTYPES),
       pre=st.sampled_from(FACTORS), two_waves=st.booleans(), zero_pad=st.booleans(), seed=st.integers(0, 2**20))
def test_gather_in_any_table(nat, numels, pad, grad_dt, rs_dt, pre, two_waves, zero_pad, seed):
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


@settings(max_examples=80, **COMMON)
@given(numels=tables, pad=st.integers(0, 700), flat_dt=st.sampled_from(DTYPES), out_dt=st.sampled_from(DTYPES),
       two_waves=st.booleans(), bound=st.booleans(), seed=st.integers(0, 2**20))
def test_scatter_out_any_table(nat, numels, pad, flat_dt, out_dt, two_waves, bound, seed):
    print("scatter_out", numels, pad, flat_dt, out_dt, two_waves, bound, seed, flush=True)
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    p, t = len(numels), sum(numels)
    flat = mixed_values(g, t + pad, flat_dt)
    modes = rng.integers(0, 2, size=p).tolist()
    offs = [int(rng.integers(0, 8)) for _ in numels]
    bufs, views = zip(*[_view_at(torch.full((n,), 3.0, dtype=out_dt), o) for n, o in zip(numels, offs)])
    default = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_TABLE_LARGE_LOG2, 0 if two_waves else default)
    try:
        table = nat.TensorTable(numels, t + pad, DEV)
    finally:
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default)
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
