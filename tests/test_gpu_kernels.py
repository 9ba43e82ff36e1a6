"""GPU parity: every C-ABI entry point against the oracle (the reference's
torch-op sequence on CPU) on the same seeded inputs, bit for bit.

Floating-point tolerance: none.  Integer views of the outputs must be equal;
the single exception is that any NaN matches any NaN (payloads are not defined
by the reference).
"""

import numpy as np
import pytest
import torch

from oracle import torch_ops
from tests.helpers import DTYPES, assert_bits_equal, mixed_values, special_values_f32

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def nat():
    from yafsdp_amd import _native

    return _native


def _say(*a):
    print(*a, flush=True)


# --------------------------------------------------------------------- casts --
def test_cast_exhaustive_high_halfword(nat):
    """Every high half-word of binary32 with low half-words straddling the tie,
    through the copy-in kernel, against the integer closed form."""
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0, 1, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x1234, 0xC000], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    x = torch.from_numpy(bits.view(np.float32).copy())
    for dt in (torch.bfloat16, torch.float16):
        _say("cast f32 ->", dt)
        want = torch.empty(x.numel(), dtype=dt)
        torch_ops.copy_in(want, x)
        got = torch.empty(x.numel(), dtype=dt, device=DEV)
        nat.flat_copy(got, x.to(DEV))
        assert_bits_equal(got, want, f"f32->{dt}")
    allh = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16)
    for dt in (torch.bfloat16, torch.float16):
        src = allh.view(dt)
        want = torch.empty(65536, dtype=torch.float32)
        torch_ops.copy_in(want, src)
        got = torch.empty(65536, dtype=torch.float32, device=DEV)
        nat.flat_copy(got, src.to(DEV))
        assert_bits_equal(got, want, f"{dt}->f32")


@pytest.mark.parametrize("src_dt", DTYPES)
@pytest.mark.parametrize("dst_dt", DTYPES)
def test_flat_copy_sizes_and_alignments(nat, src_dt, dst_dt):
    g = torch.Generator().manual_seed(100)
    for n in [0, 1, 7, 8, 9, 63, 1000, 8192, 8192 * 3 + 5, 262_147]:
        for s_off, d_off in [(0, 0), (1, 0), (0, 3), (5, 7), (8, 4)]:
            _say("flat_copy", src_dt, dst_dt, n, s_off, d_off)
            src = mixed_values(g, n + s_off, src_dt)
            want = torch.full((n + d_off + 8,), 3.0, dtype=dst_dt)
            torch_ops.copy_in(want[d_off : d_off + n], src[s_off:])
            got = torch.full((n + d_off + 8,), 3.0, dtype=dst_dt, device=DEV)
            nat.flat_copy(got[d_off : d_off + n], src.to(DEV)[s_off:])
            assert_bits_equal(got, want, f"flat_copy n={n} offs=({s_off},{d_off})")


@pytest.mark.parametrize("dt", [torch.uint8, torch.int8, torch.float8_e4m3fn, torch.float8_e5m2, torch.int32])
def test_flat_copy_of_opaque_element_types(nat, dt):
    """Same-dtype copies of element types outside the path's arithmetic (the
    all-gather dtypes of tensor-subclass parameters) are byte copies at any byte
    address: every alignment of either side modulo 16 and beyond, sizes around
    the vector and tile edges, guard bytes on both sides of the destination."""
    g = torch.Generator().manual_seed(101)
    size = torch.empty(0, dtype=dt).element_size()
    sizes = [0, 1, 2, 15, 16, 17, 31, 33, 255, 4095, 4096, 4097, 12_289, 65_536 + 3, 1_048_583]
    offs = [(0, 0), (1, 0), (0, 1), (1, 1), (3, 2), (2, 3), (15, 16), (16, 15), (7, 9), (13, 5), (32, 17)]
    if size > 1:
        sizes, offs = sizes[:10], offs[:6]
    for n in sizes:
        for s_off, d_off in offs:
            _say("flat_copy bytes", dt, n, s_off, d_off)
            raw = torch.randint(0, 256, ((n + s_off) * size,), generator=g, dtype=torch.uint8)
            src = raw.view(dt)
            want = torch.full(((n + d_off + 40) * size,), 0xA5, dtype=torch.uint8).view(dt)
            torch_ops.extension_copy_in(want[d_off : d_off + n], src[s_off:])
            got = torch.full(((n + d_off + 40) * size,), 0xA5, dtype=torch.uint8, device=DEV).view(dt)
            nat.flat_copy(got[d_off : d_off + n], src.to(DEV)[s_off:])
            assert torch.equal(got.view(torch.uint8).cpu(), want.view(torch.uint8)), (dt, n, s_off, d_off)
    # a self-copy is a no-op, a partial overlap is refused
    buf = torch.arange(100, dtype=torch.uint8, device=DEV)
    nat.flat_copy(buf[1:50], buf[1:50])
    with pytest.raises(RuntimeError):
        nat.flat_copy(buf[1:50], buf[4:53])
    assert torch.equal(buf.cpu(), torch.arange(100, dtype=torch.uint8))


def test_flat_copy_same_dtype_is_byte_copy(nat):
    # NaN payloads and every bit pattern pass through a same-dtype copy
    allh = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16)
    for dt in (torch.bfloat16, torch.float16):
        src = allh.view(dt).to(DEV)
        dst = torch.zeros_like(src)
        nat.flat_copy(dst, src)
        assert torch.equal(dst.view(torch.int16).cpu(), allh)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("factor", [None, 1.0, 0.5, 2.0, 8.0, 64.0, 256.0, 3.0, 7.0, 1.5, 1000.0, 2.0**100])
def test_flat_div(nat, dt, factor):
    g = torch.Generator().manual_seed(101)
    for n, off in [(4099, 0), (20_000, 3)]:
        _say("flat_div", dt, factor, n, off)
        x = mixed_values(g, n + off, dt, std=1e-3)
        want = x.clone()
        torch_ops.div_if_needed(want[off:], factor)
        got = x.to(DEV)
        nat.flat_div(got[off:], factor)
        assert_bits_equal(got, want, f"div {dt} {factor}")


@pytest.mark.parametrize("shard_dt", DTYPES)
@pytest.mark.parametrize("chunk_dt", DTYPES)
@pytest.mark.parametrize("post", [None, 8.0, 3.0])
@pytest.mark.parametrize("acc", [False, True])
def test_post_reduce(nat, shard_dt, chunk_dt, post, acc):
    g = torch.Generator().manual_seed(102)
    for n, off in [(5, 0), (8192 * 2 + 11, 0), (30_001, 1)]:
        _say("post_reduce", shard_dt, chunk_dt, post, acc, n, off)
        chunk = mixed_values(g, n + off, chunk_dt, std=1e-3)
        shard0 = mixed_values(g, n + off, shard_dt, std=1e-4).flip(0).contiguous()
        want = shard0.clone()
        torch_ops.reduce_scatter_local(want[off:], chunk.clone()[off:], 1, 0, None, post, "add" if acc else "copy")
        got = shard0.to(DEV)
        nat.post_reduce(got[off:], chunk.to(DEV)[off:], post, acc)
        assert_bits_equal(got, want, "post_reduce")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("scalar", [1 / 3, 1 / 5, 1 / 6, 1 / 8, 0.5, 1.0, 2.0, 1 / 1000, 1 / 7])
def test_flat_premul(nat, dt, scalar):
    """One rank's share of the collective's pre-multiplied sum, in place."""
    g = torch.Generator().manual_seed(141)
    for n, off in [(4099, 0), (20_000, 3)]:
        _say("flat_premul", dt, scalar, n, off)
        x = mixed_values(g, n + off, dt, std=1e-3)
        want = x.clone()
        torch_ops.reduce_scatter_one_rank_share(want[off:], "PREMUL_SUM", 8, scalar)
        got = x.to(DEV)
        nat.flat_premul(got[off:], scalar)
        assert_bits_equal(got, want, f"premul {dt} {scalar}")


@pytest.mark.parametrize("shard_dt", DTYPES)
@pytest.mark.parametrize("chunk_dt", DTYPES)
@pytest.mark.parametrize("op,w,factor", [("AVG", 3, None), ("AVG", 6, None), ("AVG", 8, None), ("PREMUL_SUM", 8, 3.0),
                                         ("PREMUL_SUM", 6, 5.0)])
@pytest.mark.parametrize("acc", [False, True])
def test_post_reduce_premul(nat, shard_dt, chunk_dt, op, w, factor, acc):
    g = torch.Generator().manual_seed(142)
    premul = None if factor is None else 1 / factor
    for n, off in [(5, 0), (8192 * 2 + 11, 0), (30_001, 1)]:
        _say("post_reduce_premul", shard_dt, chunk_dt, op, w, factor, acc, n, off)
        chunk = mixed_values(g, n + off, chunk_dt, std=1e-3)
        shard0 = mixed_values(g, n + off, shard_dt, std=1e-4).flip(0).contiguous()
        want = shard0.clone()
        torch_ops.reduce_scatter_local(want[off:], chunk.clone()[off:], 1, 0, None, None, "add" if acc else "copy",
                                       collective=(op, premul) if op == "PREMUL_SUM" else None)
        if op == "AVG":  # (the oracle's AVG takes the scalar from the group size: restate it with that size)
            want = shard0.clone()
            scaled = chunk.clone()
            torch_ops.reduce_scatter_one_rank_share(scaled[off:], "AVG", w)
            torch_ops.reduce_scatter_local(want[off:], scaled[off:], 1, 0, None, None, "add" if acc else "copy")
        got = shard0.to(DEV)
        d_chunk = chunk.to(DEV)
        nat.post_reduce_premul(got[off:], d_chunk[off:], 1.0 / w if op == "AVG" else premul, acc)
        assert_bits_equal(got, want, "post_reduce_premul")
        assert_bits_equal(d_chunk, chunk, "the chunk is not written")


def test_per_table_write_through_tail(nat):
    """A table's own tail option takes precedence over the process-wide one, changes no byte, and -1 hands the
    choice back."""
    g = torch.Generator().manual_seed(143)
    numels = [300_001, 7, 1_200_000, 65]
    t = sum(numels)
    t_pad = t + 183
    grads = [mixed_values(g, n, torch.bfloat16, std=1e-3) for n in numels]
    want = torch.zeros(t_pad, dtype=torch.bfloat16)
    torch_ops.reduce_copy_in(list(want[:t].split(numels)), grads, False)
    torch_ops.div_if_needed(want, 8.0)
    table = nat.TensorTable(numels, t_pad, DEV)
    d_grads = [x.to(DEV) for x in grads]
    assert table.get_option(nat.OPT_GATHER_TAIL_MB) == -1 and table.get_option(nat.OPT_SCATTER_TAIL_MB) == -1
    for mb in (0, 1, 2, 1 << 20, -1):  # 3 MB of output: the boundary lies inside the buffer for 1 and 2
        _say("per-table gather tail", mb)
        table.set_option(nat.OPT_GATHER_TAIL_MB, mb)
        assert table.get_option(nat.OPT_GATHER_TAIL_MB) == mb
        got = torch.full((t_pad,), 9.0, dtype=torch.bfloat16, device=DEV)
        table.gather_in(d_grads, got, None, 8.0, True)
        assert_bits_equal(got, want, f"gather_in with a table tail of {mb} MB")
        table.set_option(nat.OPT_SCATTER_TAIL_MB, mb)
        outs = [torch.empty(n, dtype=torch.bfloat16, device=DEV) for n in numels]
        table.scatter_out(got, outs)
        for a, b in zip(outs, want[:t].split(numels)):
            assert_bits_equal(a, b, f"scatter_out with a table tail of {mb} MB")
    with pytest.raises(RuntimeError):
        table.set_option(nat.OPT_FLAT_TAIL_MB, 1)  # only the two table kernels' tails are per table
    assert nat.get_store_policy() == nat.STORE_POLICIES["rotating_sets"]  # the process-wide options were not touched
    table.close()


@pytest.mark.parametrize("tail_mb", [0, 1, 3, 1 << 20])
def test_flat_kernels_with_the_write_through_boundary_inside_the_buffer(nat, tail_mb):
    """The flat kernels store non-temporal by default (tail option 0); with a tail option below the size of the output
    the last megabytes are stored write-through instead (2^20: everything).  Same bytes either way."""
    g = torch.Generator().manual_seed(131)
    n = 1_500_003  # 3 MB of bf16, 6 MB of fp32
    defaults = (nat.get_option(nat.OPT_FLAT_TAIL_MB), nat.get_option(nat.OPT_POST_REDUCE_TAIL_MB))
    nat.set_option(nat.OPT_FLAT_TAIL_MB, tail_mb)
    nat.set_option(nat.OPT_POST_REDUCE_TAIL_MB, tail_mb)
    try:
        for src_dt, dst_dt in [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32),
                               (torch.bfloat16, torch.bfloat16)]:
            _say("flat_copy with tail", tail_mb, src_dt, dst_dt)
            src = mixed_values(g, n + 1, src_dt)
            want = torch.full((n + 11,), 3.0, dtype=dst_dt)
            torch_ops.copy_in(want[3 : 3 + n], src[1:])
            got = torch.full((n + 11,), 3.0, dtype=dst_dt, device=DEV)
            nat.flat_copy(got[3 : 3 + n], src.to(DEV)[1:])
            assert_bits_equal(got, want, "flat_copy")
        raw = torch.randint(0, 256, (4 * n + 8,), generator=g, dtype=torch.uint8)  # 6 MB between odd byte addresses
        got = torch.zeros(4 * n + 8, dtype=torch.uint8, device=DEV)
        nat.flat_copy(got[3 : 3 + 4 * n], raw.to(DEV)[1 : 1 + 4 * n])
        assert torch.equal(got[3 : 3 + 4 * n].cpu(), raw[1 : 1 + 4 * n]) and int(got[:3].max()) == 0
        assert int(got[3 + 4 * n :].max()) == 0
        buf = mixed_values(g, n, torch.bfloat16)
        want = buf.clone()
        torch_ops.div_if_needed(want, 8.0)
        got = buf.to(DEV)
        nat.flat_div(got, 8.0)
        assert_bits_equal(got, want, "flat_div")
        for acc in (False, True):
            _say("post_reduce with tail", tail_mb, acc)
            chunk = mixed_values(g, n, torch.bfloat16, std=1e-3)
            shard0 = mixed_values(g, n, torch.float32, std=1e-4)
            want = shard0.clone()
            torch_ops.reduce_scatter_local(want, chunk.clone(), 1, 0, None, 8.0, "add" if acc else "copy")
            got = shard0.to(DEV)
            nat.post_reduce(got, chunk.to(DEV), 8.0, acc)
            assert_bits_equal(got, want, "post_reduce")
    finally:
        nat.set_option(nat.OPT_FLAT_TAIL_MB, defaults[0])
        nat.set_option(nat.OPT_POST_REDUCE_TAIL_MB, defaults[1])


@pytest.mark.parametrize("shard_dt,chunk_dt", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("post", [None, 8.0])
def test_post_reduce_fragments(nat, shard_dt, chunk_dt, post):
    g = torch.Generator().manual_seed(103)
    numels = [0, 7, 12_001, 0, 33, 1, 9000, 5]
    has = [None, True, False, False, None, True, True, None]
    s = sum(numels) + 16
    chunk = mixed_values(g, s, chunk_dt, 1e-3)
    shard0 = mixed_values(g, s, shard_dt, 1e-4).flip(0).contiguous()
    want = shard0.clone()
    torch_ops.reduce_scatter_local(want, chunk.clone(), 1, 0, None, post, "mixed", numels, has)
    got = shard0.to(DEV)
    modes = [0 if h is None else (2 if h else 1) for h in has]
    nat.post_reduce_fragments(got, chunk.to(DEV), numels, modes, post)
    assert_bits_equal(got, want, "post_reduce_fragments")


# ------------------------------------------------------------- table kernels --
def _random_numels(rng: np.random.Generator, p: int, max_log2: float, with_empty: bool):
    n = np.floor(np.exp2(rng.uniform(0, max_log2, size=p))).astype(np.int64) | 1
    if with_empty and p > 3:
        n[rng.integers(0, p, size=max(1, p // 10))] = 0
    return n.tolist()


@pytest.fixture(params=["one_wave", "two_waves", "short_scatter_tiles"])
def table_workgroup(request, nat):
    """Run a table test at both workgroup sizes the library picks between by table size, and with the short
    scatter-out tile it picks for tables whose tensors all start on a cache line."""
    default = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_TABLE_LARGE_LOG2, 0 if request.param == "two_waves" else default)
    nat.set_option(nat.OPT_SCATTER_TILE, 1 if request.param == "short_scatter_tiles" else 2)
    yield request.param
    nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default)
    nat.set_option(nat.OPT_SCATTER_TILE, 0)


TABLE_CASES = [
    # (P, max log2 numel, with_empty, pad)
    (1, 3, False, 0),
    (3, 4, False, 5),
    (9, 16, True, 17),
    (32, 14, True, 0),
    (33, 14, True, 9),
    (200, 12, True, 4096),
    (40, 19, False, 513),
]


@pytest.mark.parametrize("case", TABLE_CASES)
@pytest.mark.parametrize("grad_dt,rs_dt", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                           (torch.float32, torch.bfloat16), (torch.float16, torch.float16),
                                           (torch.float32, torch.float32)])
@pytest.mark.parametrize("pre", [None, 8.0, 3.0])
def test_gather_in(nat, table_workgroup, case, grad_dt, rs_dt, pre):
    _check_gather_in(nat, case, grad_dt, rs_dt, pre)


@pytest.mark.parametrize("tail_mb", [0, 1, 3])
@pytest.mark.parametrize("large_log2", [None, 0])
@pytest.mark.parametrize("grad_dt,rs_dt,pre", [(torch.bfloat16, torch.bfloat16, None),
                                               (torch.float32, torch.bfloat16, 8.0),
                                               (torch.bfloat16, torch.float32, 3.0)])
def test_gather_in_with_the_write_through_boundary_inside_the_buffer(nat, tail_mb, large_log2, grad_dt, rs_dt, pre):
    """The last megabytes of the flat buffer are stored with another cache policy than the rest (0: none are; the
    default is larger than any buffer of these tests, so everywhere else all tiles are).  Same bytes either way."""
    default_tail = nat.get_option(nat.OPT_GATHER_TAIL_MB)
    default_log2 = nat.get_option(nat.OPT_TABLE_LARGE_LOG2)
    nat.set_option(nat.OPT_GATHER_TAIL_MB, tail_mb)
    if large_log2 is not None:
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, large_log2)
    try:
        for case in [(40, 19, False, 513), (33, 14, True, 9), (9, 21, False, 17)]:
            _check_gather_in(nat, case, grad_dt, rs_dt, pre)
    finally:
        nat.set_option(nat.OPT_GATHER_TAIL_MB, default_tail)
        nat.set_option(nat.OPT_TABLE_LARGE_LOG2, default_log2)


def _check_gather_in(nat, case, grad_dt, rs_dt, pre):
    p, max_log2, with_empty, pad = case
    rng = np.random.default_rng(p * 1000 + pad)
    g = torch.Generator().manual_seed(104 + p)
    numels = _random_numels(rng, p, max_log2, with_empty)
    t = sum(numels)
    t_pad = t + pad
    _say("gather_in", case, grad_dt, rs_dt, pre, "T", t)
    grads = [mixed_values(g, n, grad_dt, 1e-3) for n in numels]
    modes = rng.integers(0, 3, size=p).tolist() if p > 1 else [1]
    old = torch.zeros(t_pad + 8, dtype=rs_dt)
    old[:t] = mixed_values(g, t, rs_dt, 1e-3).flip(0)
    old[t_pad:] = 5.0  # guard lanes beyond the padded buffer stay untouched
    # oracle: foreach copy, foreach add, then div over the padded buffer
    want = old.clone()
    views = list(want[:t].split(numels))
    cp = [i for i, m in enumerate(modes) if m == 1]
    ad = [i for i, m in enumerate(modes) if m == 2]
    torch_ops.reduce_copy_in([views[i] for i in cp], [grads[i] for i in cp], False)
    torch_ops.reduce_copy_in([views[i] for i in ad], [grads[i] for i in ad], True)
    torch_ops.div_if_needed(want[:t_pad], pre)
    table = nat.TensorTable(numels, t_pad, torch.device(DEV))
    got = old.to(DEV)
    # sources start at odd element offsets of their allocations (views, as gradients of sliced parameters are)
    dgrads = [torch.cat([x.new_zeros(i % 5), x]).to(DEV)[i % 5 :] for i, x in enumerate(grads)]
    table.gather_in(dgrads, got, modes, pre, zero_pad=True)
    assert_bits_equal(got, want, "gather_in")
    # all-copy call with default modes
    want2 = old.clone()
    torch_ops.reduce_copy_in(list(want2[:t].split(numels)), grads, False)
    got2 = old.to(DEV)
    table.gather_in(dgrads, got2)
    assert_bits_equal(got2, want2, "gather_in all copy")
    table.close()


def test_gather_in_pad_not_zeroed_sees_divide(nat):
    numels = [100, 29]
    t, t_pad = 129, 160
    g = torch.Generator().manual_seed(105)
    old = mixed_values(g, t_pad, torch.bfloat16, 1e-2)
    grads = [mixed_values(g, n, torch.bfloat16, 1e-3) for n in numels]
    want = old.clone()
    torch_ops.reduce_copy_in(list(want[:t].split(numels)), grads, False)
    torch_ops.div_if_needed(want, 4.0)
    table = nat.TensorTable(numels, t_pad, torch.device(DEV))
    got = old.to(DEV)
    table.gather_in([x.to(DEV) for x in grads], got, None, 4.0, zero_pad=False)
    assert_bits_equal(got, want, "pad lanes divided like the reference's")


@pytest.mark.parametrize("case", TABLE_CASES)
@pytest.mark.parametrize("flat_dt,out_dt", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32),
                                            (torch.bfloat16, torch.float32), (torch.float32, torch.float16)])
def test_scatter_out(nat, table_workgroup, case, flat_dt, out_dt):
    p, max_log2, with_empty, pad = case
    rng = np.random.default_rng(p * 1000 + pad + 1)
    g = torch.Generator().manual_seed(106 + p)
    numels = _random_numels(rng, p, max_log2, with_empty)
    t = sum(numels)
    _say("scatter_out", case, flat_dt, out_dt, "T", t)
    flat = mixed_values(g, t + pad, flat_dt)
    want = [torch.full((n + 2,), 3.0, dtype=out_dt) for n in numels]
    torch_ops.copy_out_materialize(flat, numels, [w[1 : 1 + n] for w, n in zip(want, numels)])
    got = [torch.full((n + 2,), 3.0, dtype=out_dt, device=DEV) for n in numels]
    table = nat.TensorTable(numels, t + pad, torch.device(DEV))
    table.scatter_out(flat.to(DEV), [x[1 : 1 + n] for x, n in zip(got, numels)])
    for i, (a, b) in enumerate(zip(got, want)):
        assert_bits_equal(a, b, f"scatter_out tensor {i}")
    # skip modes: untouched outputs
    if p > 1:
        modes = rng.integers(0, 2, size=p).tolist()
        got2 = [torch.full((n,), 3.0, dtype=out_dt, device=DEV) for n in numels]
        table.scatter_out(flat.to(DEV), got2, modes)
        pos = 0
        for i, n in enumerate(numels):
            ref = torch.full((n,), 3.0, dtype=out_dt)
            if modes[i]:
                ref.copy_(flat[pos : pos + n])
            assert_bits_equal(got2[i], ref, f"scatter_out modes tensor {i}")
            pos += n
    table.close()


@pytest.mark.parametrize("case", [TABLE_CASES[1], TABLE_CASES[4], TABLE_CASES[5]])
def test_bound_calls_match_per_call_pointers(nat, table_workgroup, case):
    """A binding fixes pointers, modes and dtype once; bound launches give the same bits as per-call ones,
    call after call, for tables that travel in the kernel arguments and for staged ones."""
    p, max_log2, with_empty, pad = case
    rng = np.random.default_rng(p * 77 + pad)
    g = torch.Generator().manual_seed(140 + p)
    numels = _random_numels(rng, p, max_log2, with_empty)
    t = sum(numels)
    t_pad = t + pad
    modes = rng.integers(0, 3, size=p).tolist()
    grads = [mixed_values(g, n, torch.bfloat16, 1e-3).to(DEV) for n in numels]
    old = mixed_values(g, t_pad, torch.float32, 1e-3)
    table = nat.TensorTable(numels, t_pad, torch.device(DEV))
    want = old.to(DEV)
    table.gather_in(grads, want, modes, 3.0, True)
    binding = table.bind(grads, modes)
    for _ in range(2):
        got = old.to(DEV)
        binding.gather_in(got, 3.0, True)
        assert_bits_equal(got, want, "bound gather_in")
    # the tensors' contents may change between calls, their addresses may not
    for x in grads:
        x.mul_(2)
    table.gather_in(grads, want := old.to(DEV), modes, None, True)
    binding.gather_in(got := old.to(DEV), None, True)
    assert_bits_equal(got, want, "bound gather_in after the tensors changed")
    # scatter
    flat = mixed_values(g, t_pad, torch.bfloat16).to(DEV)
    smodes = [int(m > 0) for m in modes]
    outs_a = [torch.full((n,), 3.0, dtype=torch.float32, device=DEV) for n in numels]
    outs_b = [torch.full((n,), 3.0, dtype=torch.float32, device=DEV) for n in numels]
    table.scatter_out(flat, outs_a, smodes)
    sb = table.bind(outs_b, smodes)
    sb.scatter_out(flat)
    for i, (a, b) in enumerate(zip(outs_a, outs_b)):
        assert_bits_equal(b, a, f"bound scatter_out tensor {i}")
    with pytest.raises(ValueError):
        table.bind(grads[:-1])
    sb.close(), binding.close(), table.close()


def test_errors_are_loud(nat):
    a = torch.zeros(16, dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError):
        nat.flat_copy(a, torch.zeros(16))  # CPU tensor: no CPU path
    with pytest.raises(TypeError):
        nat.flat_copy(a, torch.zeros(16, dtype=torch.float64, device=DEV))
    with pytest.raises(ValueError):
        nat.flat_copy(a, torch.zeros(8, device=DEV))
    with pytest.raises(NotImplementedError):
        nat.flat_copy(a.view(4, 4).t(), a.view(4, 4))
    table = nat.TensorTable([8, 8], 16, torch.device(DEV))
    with pytest.raises(ValueError):
        table.gather_in([a[:8]], a.bfloat16())
    with pytest.raises(RuntimeError, match="aligned"):
        buf = torch.zeros(32, dtype=torch.bfloat16, device=DEV)
        table.gather_in([a[:8], a[8:]], buf[1:17])
    assert "invalid argument" in nat.error_string(-1)
    assert nat.lib.yafsdp_flat_copy(a.data_ptr(), 7, a.data_ptr(), 0, 4, None) == -2


def test_time_next_launch_brackets_exactly_one_dispatch(nat):
    """Events armed with time_next_launch ride on the next dispatch only: the measured time is that kernel's
    own duration (shorter than a record / launch / record bracket) and results are unchanged."""
    n = 1 << 26
    src = torch.randn(n, device=DEV)
    dst = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(3):
        nat.flat_copy(dst, src)
    nat.time_next_launch(a, b)
    nat.flat_copy(dst, src)
    small = torch.empty(8, dtype=torch.bfloat16, device=DEV)
    nat.flat_copy(small, src[:8])  # not timed: the pair was consumed
    torch.cuda.synchronize()
    attached = a.elapsed_time(b) * 1e3
    c, d = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c.record()
    nat.flat_copy(dst, src)
    d.record()
    torch.cuda.synchronize()
    bracket = c.elapsed_time(d) * 1e3
    _say("attached", attached, "bracket", bracket)
    assert 20.0 < attached < 500.0  # 403 MB: about 65 us at 6 TB/s
    assert attached <= bracket + 2.0
    assert_bits_equal(dst, src.bfloat16(), "timed launch result")
    nat.time_next_launch(a, b)
    nat.time_next_launch(None, None)  # disarm
    nat.flat_copy(dst, src)
    torch.cuda.synchronize()
    assert abs(a.elapsed_time(b) * 1e3 - attached) < 1e-6  # untouched by the disarmed launch


def test_table_with_the_maximum_number_of_tensors(nat):
    """65,534 tensors of 0-5 elements (the reference allows fewer than 65,535 parameters per group,
    ya_fsdp/_param_group.py:284-287): almost every tile crosses many tensor boundaries."""
    p = 65_534
    rng = np.random.default_rng(9)
    numels = rng.integers(0, 6, size=p).tolist()
    t = sum(numels)
    t_pad = t + 11
    g = torch.Generator().manual_seed(150)
    src = mixed_values(g, t, torch.bfloat16, 1e-3)
    grads = list(src.split(numels))
    old = mixed_values(g, t_pad, torch.float32, 1e-3)
    want = old.clone()
    torch_ops.reduce_copy_in(list(want[:t].split(numels)), grads, False)
    want[t:] = 0
    torch_ops.div_if_needed(want, 8.0)
    dsrc = src.to(DEV)
    dgrads = list(dsrc.split(numels))
    table = nat.TensorTable(numels, t_pad, torch.device(DEV))
    got = old.to(DEV)
    table.gather_in(dgrads, got, None, 8.0, True)
    assert_bits_equal(got, want, "gather_in, 65,534 tensors")
    flat = mixed_values(g, t_pad, torch.float32).to(DEV)
    out = torch.zeros(t, dtype=torch.bfloat16, device=DEV)
    table.scatter_out(flat, list(out.split(numels)))
    assert_bits_equal(out, flat[:t].cpu().bfloat16(), "scatter_out, 65,534 tensors")
    table.close()


def test_completion_event_recorded_by_the_launch_itself(nat):
    """``launch_recording``: the kernel's own dispatch records the event.  Another stream that waits for the event
    sees the kernel's output (new data every round, so a missed dependency shows as stale values), the host can
    synchronise on it, and a call that launches nothing still leaves the event recorded."""
    g = torch.Generator().manual_seed(151)
    n = 8_000_000
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    event = torch.cuda.Event()
    src = torch.empty(n, dtype=torch.float32, device=DEV)
    mid = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
    out = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
    main = torch.cuda.current_stream()
    for round_ in range(6):
        _say("completion event round", round_)
        x = torch.randn(n, generator=g) * 0.02 + round_
        src.copy_(x.to(DEV))
        a.wait_stream(main)
        with torch.cuda.stream(a):
            got = nat.launch_recording(event, lambda: nat.flat_copy(mid, src), a)
            assert got is event
        with torch.cuda.stream(b):
            b.wait_event(event)
            nat.flat_copy(out, mid)
        main.wait_stream(b)
        assert_bits_equal(out, x.bfloat16(), f"round {round_}")
        b.wait_stream(main)
        a.wait_stream(main)  # the next round's src.copy_ must not overtake this round's reads
    with torch.cuda.stream(a):
        src.fill_(3.0)
        nat.launch_recording(event, lambda: nat.flat_copy(mid, src), a)
    event.synchronize()  # the host waits for the kernel through the same event
    assert event.query() and float(mid[n - 1]) == 3.0 and float(mid[0]) == 3.0
    # nothing to launch: the event is recorded the ordinary way, and nothing stays armed for a later launch
    fresh = torch.cuda.Event()
    with torch.cuda.stream(a):
        nat.launch_recording(fresh, lambda: nat.flat_copy(mid[:0], src[:0]), a)
    fresh.synchronize()
    assert fresh.query() and nat.lib.yafsdp_complete_next_launch_pending() == 0
