"""Pin the oracle: the torch-op sequence (oracle.torch_ops) against closed forms,
hand-checked cases, numpy float64 arithmetic rounded once, and the independent
plain-C restatement (oracle.cref)."""

import numpy as np
import pytest
import torch

from oracle import cref, torch_ops
from tests.helpers import DTYPES, assert_bits_equal, mixed_values, special_values_f32


def _bf16_closed_form(bits: np.ndarray) -> np.ndarray:
    bits = bits.astype(np.uint64)
    return (((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def test_bf16_cast_hand_checked_ties():
    # 1 + 2^-8 is a tie between 0x3F80 and 0x3F81 -> even 0x3F80; 1 + 3*2^-8 -> 0x3F82
    x = torch.tensor([1 + 2**-8, 1 + 3 * 2**-8, -0.0, 2.0**-130], dtype=torch.float32)
    out = torch.empty(4, dtype=torch.bfloat16)
    torch_ops.copy_in(out, x)
    got = out.view(torch.int16).numpy().view(np.uint16).tolist()
    sub = np.array([2.0**-130], dtype=np.float32).view(np.uint32)[0]
    assert got[:3] == [0x3F80, 0x3F82, 0x8000]
    assert got[3] == int(_bf16_closed_form(np.array([sub]))[0]) and got[3] != 0  # subnormal kept
    for v, g in zip(x.view(torch.int32).tolist(), got):
        assert cref.lib().ref_f32_to_bf16(v & 0xFFFFFFFF) == g


def test_bf16_cast_closed_form_random_and_exhaustive_high_bits():
    g = torch.Generator().manual_seed(7)
    # every high half-word with a set of low half-words that straddle the tie
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0, 1, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    rnd = torch.randint(0, 2**31 - 1, (1 << 18,), generator=g, dtype=torch.int64).numpy().astype(np.uint32) * 2
    bits = np.concatenate([bits, rnd])
    x = torch.from_numpy(bits.view(np.float32).copy())
    out = torch.empty(x.numel(), dtype=torch.bfloat16)
    torch_ops.copy_in(out, x)
    got = out.view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(bits.view(np.float32))
    want = _bf16_closed_form(bits)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(out.float().numpy()[nan]).all()
    # C restatement on the same inputs
    out_c = torch.empty_like(out)
    cref.flat_copy(out_c, x)
    assert_bits_equal(out_c, out, "C vs torch f32->bf16")


def test_f16_cast_vs_numpy_and_c():
    g = torch.Generator().manual_seed(8)
    x = torch.cat([special_values_f32(), mixed_values(g, 1 << 16, torch.float32, std=1.0),
                   torch.randn(1 << 16, generator=g) * 1e-6, torch.randn(1 << 12, generator=g) * 7e4])
    out = torch.empty(x.numel(), dtype=torch.float16)
    torch_ops.copy_in(out, x)
    with np.errstate(over="ignore"):
        want = torch.from_numpy(x.numpy().astype(np.float16))
    assert_bits_equal(out, want, "torch vs numpy f32->f16")
    out_c = torch.empty_like(out)
    cref.flat_copy(out_c, x)
    assert_bits_equal(out_c, out, "C vs torch f32->f16")
    # widening is exact, for every half-precision pattern
    allh = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16)
    for dt in (torch.float16, torch.bfloat16):
        src = allh.view(dt)
        a, b = torch.empty(65536, dtype=torch.float32), torch.empty(65536, dtype=torch.float32)
        torch_ops.copy_in(a, src)
        cref.flat_copy(b, src)
        assert_bits_equal(a, b, f"widen {dt}")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("factor", [2.0, 8.0, 64.0, 3.0, 7.0, 1.5, 1.0, 0.5, 1000.0])
def test_div_is_true_binary32_division(dt, factor):
    g = torch.Generator().manual_seed(11)
    x = mixed_values(g, 1 << 15, dt, std=1e-3)
    a = x.clone()
    torch_ops.div_if_needed(a, factor)
    b = x.clone()
    cref.flat_div(b, factor)
    assert_bits_equal(a, b, "div_ torch vs C")
    if factor <= 1:
        assert_bits_equal(a, x, "factor <= 1 is skipped")  # ya_fsdp/_collectives.py:271
        return
    # float64 quotient of two binary32 numbers rounded once to binary32 is the
    # correctly rounded binary32 quotient (53 >= 2*24+2), then round to dt
    finite = torch.isfinite(x.float())
    q = (x.double() / float(np.float32(factor))).float().to(dt)
    assert_bits_equal(a[finite], q[finite], "div_ vs float64")


@pytest.mark.parametrize("shard_dt,chunk_dt", [(torch.float32, torch.bfloat16), (torch.float32, torch.float32),
                                               (torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16),
                                               (torch.float32, torch.float16), (torch.float16, torch.float16)])
@pytest.mark.parametrize("post", [None, 8.0, 3.0])
@pytest.mark.parametrize("acc", [False, True])
def test_post_reduce_rounding_order(shard_dt, chunk_dt, post, acc):
    g = torch.Generator().manual_seed(13)
    n = 1 << 14
    chunk = mixed_values(g, n, chunk_dt, std=1e-3)
    shard0 = mixed_values(g, n, shard_dt, std=1e-4).flip(0).contiguous()
    # torch-op sequence on a W=1 "buffer"
    shard_t, buf = shard0.clone(), chunk.clone()
    torch_ops.reduce_scatter_local(shard_t, buf, 1, 0, None, post, "add" if acc else "copy")
    shard_c = shard0.clone()
    cref.post_reduce(shard_c, chunk, post, acc)
    assert_bits_equal(shard_t, shard_c, "post-reduce torch vs C")
    # independent: float64 arithmetic with one rounding per materialised tensor
    y = chunk.double()
    if post is not None:
        y = (y / float(np.float32(post))).float().to(chunk_dt).double()
    if acc:
        y = shard0.double() + y
    want = y.float().to(shard_dt)
    ok = torch.isfinite(want.float()) & torch.isfinite(chunk.float()) & torch.isfinite(shard0.float())
    assert_bits_equal(shard_t[ok], want[ok], "post-reduce vs float64")


@pytest.mark.parametrize("grad_dt,rs_dt", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                           (torch.float32, torch.bfloat16), (torch.float16, torch.float16),
                                           (torch.float32, torch.float32)])
@pytest.mark.parametrize("pre", [None, 8.0, 3.0])
def test_gather_in_copy_add_skip_vs_c(grad_dt, rs_dt, pre):
    g = torch.Generator().manual_seed(17)
    numels = [5, 1, 300, 0, 77, 1024, 3]
    t = sum(numels)
    t_pad = t + 6
    offsets = np.concatenate([[0], np.cumsum(numels)])
    grads = [mixed_values(g, n, grad_dt, 1e-3) for n in numels]
    modes = [1, 2, 1, 1, 0, 2, 2]
    old = torch.zeros(t_pad, dtype=rs_dt)
    old[:t] = mixed_values(g, t, rs_dt, 1e-3).flip(0)
    # torch-op sequence
    flat_t = old.clone()
    views = list(flat_t[:t].split(numels))
    torch_ops.reduce_copy_in([views[i] for i, m in enumerate(modes) if m == 1], [grads[i] for i, m in enumerate(modes) if m == 1], False)
    torch_ops.reduce_copy_in([views[i] for i, m in enumerate(modes) if m == 2], [grads[i] for i, m in enumerate(modes) if m == 2], True)
    torch_ops.div_if_needed(flat_t, pre)
    flat_c = old.clone()
    cref.gather_in(grads, modes, offsets, flat_c, t_pad, pre, True)
    assert_bits_equal(flat_t, flat_c, "gather-in torch vs C")
    assert (flat_t[t:] == 0).all()


def test_scatter_out_is_byte_identity_and_views_alias():
    g = torch.Generator().manual_seed(19)
    numels = [12, 1, 35, 8]
    sizes = [(3, 4), (1,), (5, 7), (2, 2, 2)]
    flat = mixed_values(g, sum(numels) + 8, torch.bfloat16)
    views = torch_ops.unsharded_views(flat, numels, sizes)
    assert [tuple(v.shape) for v in views] == sizes
    assert views[2].data_ptr() == flat.data_ptr() + 13 * 2  # zero-copy
    outs = [torch.empty(s, dtype=torch.bfloat16) for s in sizes]
    torch_ops.copy_out_materialize(flat, numels, outs)
    outs_c = [torch.empty(s, dtype=torch.bfloat16) for s in sizes]
    cref.scatter_out(outs_c, np.concatenate([[0], np.cumsum(numels)]), flat)
    pos = 0
    for o, oc, n in zip(outs, outs_c, numels):
        assert_bits_equal(o.view(-1), flat[pos : pos + n], "split+copy_")
        assert_bits_equal(oc, o, "C scatter")
        pos += n


def test_pre_then_post_divide_chain_matches_fused_reading():
    """grad -> cast rs -> /pre (round rs) -> chunk -> /post (round rs) -> fp32 add."""
    g = torch.Generator().manual_seed(23)
    w, r, s = 4, 2, 256
    grads = mixed_values(g, w * s, torch.float16, 1e-2)
    shard0 = mixed_values(g, s, torch.float32, 1e-4)
    buf = torch.zeros(w * s, dtype=torch.float16)
    torch_ops.reduce_copy_in([buf], [grads], False)
    shard = shard0.clone()
    torch_ops.reduce_scatter_local(shard, buf, w, r, 2.0, 2.0, "add")
    buf_c = torch.zeros(w * s, dtype=torch.float16)
    cref.gather_in([grads], [1], [0, w * s], buf_c, w * s, 2.0, True)
    shard_c = shard0.clone()
    cref.post_reduce(shard_c, buf_c[r * s : (r + 1) * s].clone(), 2.0, True)
    assert_bits_equal(shard, shard_c, "chain")


def test_mixed_fragments():
    g = torch.Generator().manual_seed(29)
    sharded_numels = [0, 7, 120, 0, 33]
    s = sum(sharded_numels) + 8
    chunk_src = mixed_values(g, s, torch.bfloat16, 1e-3)
    shard0 = mixed_values(g, s, torch.float32, 1e-4)
    has = [None, True, False, False, None]
    shard = shard0.clone()
    torch_ops.reduce_scatter_local(shard, chunk_src.clone(), 1, 0, None, 8.0, "mixed", sharded_numels, has)
    want = shard0.clone()
    q = chunk_src.clone()
    cref.flat_div(q, 8.0)
    want[0:7] = shard0[0:7] + q[0:7].float()
    want[7:127] = q[7:127].float()
    assert_bits_equal(shard, want, "mixed")
    assert_bits_equal(shard[127:], shard0[127:], "untouched fragments and pad")


# ---- the collective's own scaling for group sizes above one (ya_fsdp/_collectives.py:243-249, 152-162) ----------
def _scalar_in(dt, scalar):
    """The pre-multiplier as the collective sees it: binary64 -> binary32 -> data type (by integer arithmetic for
    bf16, numpy for fp16), as a binary64 number."""
    f = np.float32(scalar)
    if dt == torch.float32:
        return float(f)
    if dt == torch.float16:
        return float(np.float16(f))
    bits = _bf16_closed_form(np.array([f], dtype=np.float32).view(np.uint32))
    return float((bits.astype(np.uint32) << 16).view(np.float32)[0])


def test_premul_scalars_hand_checked():
    # 1/3 = 0.0101010101...b: binary32 0x3EAAAAAB (rounded up), bf16 0x3EAB, fp16 0x3555
    assert np.array([_scalar_in(torch.float32, 1 / 3)], dtype=np.float32).view(np.uint32)[0] == 0x3EAAAAAB
    assert _scalar_in(torch.bfloat16, 1 / 3) == 0.333984375        # 0x3EAB
    assert _scalar_in(torch.float16, 1 / 3) == 0.333251953125      # 0x3555
    for dt, three_thirds in ((torch.bfloat16, 1.0), (torch.float16, 1.0), (torch.float32, 1.0)):
        # 3 * round(1/3) lies within half an ulp of 1 in all three types
        x = torch.tensor([1.0, 3.0, -3.0, 0.0], dtype=dt)
        torch_ops.reduce_scatter_one_rank_share(x, "AVG", 3)
        assert x.double().tolist() == [_scalar_in(dt, 1 / 3), three_thirds, -three_thirds, 0.0]
    # a case where multiplying by the rounded reciprocal and dividing part ways, by hand:
    # bf16 7.0 * 0.333984375 = 2.337890625 -> between 2.328125 (0x4015) and 2.34375 (0x4016), nearer the latter;
    # 7 / 3 = 2.3333... -> nearer 2.328125
    x = torch.tensor([7.0], dtype=torch.bfloat16)
    torch_ops.reduce_scatter_one_rank_share(x, "PREMUL_SUM", 8, 1 / 3)
    assert x.item() == 2.34375 and (torch.tensor([7.0], dtype=torch.bfloat16) / 3).item() == 2.328125


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op,w,factor", [("AVG", 3, None), ("AVG", 6, None), ("AVG", 8, None), ("AVG", 7, None),
                                         ("PREMUL_SUM", 8, 3.0), ("PREMUL_SUM", 6, 5.0), ("PREMUL_SUM", 3, 0.5),
                                         ("PREMUL_SUM", 4, 1000.0), ("SUM", 8, None)])
def test_one_rank_share_of_the_collective_is_a_rounded_product(dt, op, w, factor):
    g = torch.Generator().manual_seed(17)
    x = mixed_values(g, 1 << 15, dt, std=1e-3)
    premul = None if factor is None else 1 / factor  # what _make_nccl_premul_sum receives (:249)
    a = x.clone()
    torch_ops.reduce_scatter_one_rank_share(a, op, w, premul)
    if op == "SUM":
        assert_bits_equal(a, x, "a sum of one contribution")
        return
    scalar = 1.0 / w if op == "AVG" else premul
    b = x.clone()
    cref.flat_premul(b, scalar)
    assert_bits_equal(a, b, "pre-multiplied share: torch vs C")
    # independent: the binary64 product of two binary32 numbers is exact (48 <= 53 bits), so rounding it once to
    # binary32 gives the correctly rounded binary32 product; for the 16-bit types that product is already exact in
    # binary32 and the one rounding is the cast to the type
    k = _scalar_in(dt, scalar)
    want = (x.double() * k).float().to(dt)
    finite = torch.isfinite(x.float()) & torch.isfinite(want.float())
    assert_bits_equal(a[finite], want[finite], "pre-multiplied share vs float64")
    # and it is NOT the division that a sum followed by "/ factor" would give, unless the factor is a power of two
    f = float(w) if op == "AVG" else factor
    d = x.clone()
    d.div_(f)
    differs = int(((a.view(torch.int16 if dt != torch.float32 else torch.int32)
                    != d.view(torch.int16 if dt != torch.float32 else torch.int32)) & finite).sum())
    if f in (0.5, 8.0):
        assert differs == 0
    else:
        assert differs > 100, (op, w, factor, differs)


def test_fanin_with_premultiplied_contributions_hand_checked():
    """Three ranks, bf16, AVG: every rank's element times bf16(1/3) = 0.333984375, rounded to bf16, then added in
    binary32 in rank order and rounded to bf16 - not (a + b + c) / 3."""
    # 7 * k = 2.337890625 -> 2.34375;  1 * k -> 0.333984375;  3 * k = 1.001953125 -> 1.0 (half an ulp of 1 is 0.00390625)
    chunks = [torch.tensor([7.0, 1.0], dtype=torch.bfloat16), torch.tensor([1.0, 1.0], dtype=torch.bfloat16),
              torch.tensor([3.0, 1.0], dtype=torch.bfloat16)]
    shard = torch.zeros(2, dtype=torch.float32)
    torch_ops.reduce_scatter_fanin(shard, chunks, None, False, premul=1 / 3)
    # element 0: 2.34375 + 0.333984375 + 1.0 = 3.677734375 -> bf16 spacing 0.015625 at 2..4: 3.671875 | 3.6875, nearer 3.671875
    # element 1: 3 * 0.333984375 = 1.001953125 -> 1.0
    assert shard.tolist() == [3.671875, 1.0]
    # the sum-then-divide form gives 11 / 3 = 3.6666 -> 3.671875 as well for element 0, but differs on, e.g., 7 alone:
    lone = torch.zeros(1, dtype=torch.bfloat16)
    torch_ops.reduce_scatter_fanin(lone, [torch.tensor([7.0], dtype=torch.bfloat16)], None, False, premul=1 / 3)
    assert lone.item() == 2.34375
    other = torch.zeros(1, dtype=torch.bfloat16)
    torch_ops.reduce_scatter_fanin(other, [torch.tensor([7.0], dtype=torch.bfloat16)], 3.0, False)
    assert other.item() == 2.328125


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n_src,scalar", [(3, 1 / 3), (6, 1 / 6), (8, 1 / 8), (5, 1 / 3.0)])
def test_fanin_with_premultiplied_contributions_vs_float64(dt, n_src, scalar):
    """Independent restatement: term = the exact binary64 product rounded once to the data type (through binary32
    for the 16-bit types, where it is exact); sum = binary32 additions in rank order, each the correctly rounded
    binary64 sum of two binary32 numbers rounded once more to binary32 - which double rounding cannot change,
    because 53 >= 2 * 24 + 2; output rounded to the data type; with one contribution it is the one-rank share."""
    g = torch.Generator().manual_seed(23)
    n = 1 << 14
    chunks = [mixed_values(g, n, dt, std=1e-3, specials=False) for _ in range(n_src)]
    k = _scalar_in(dt, scalar)
    acc = None
    for c in chunks:
        term = (c.double() * k).float().to(dt).double()
        acc = term if acc is None else (acc + term).float().double()
    want = acc.float().to(dt)
    for shard_dt in (torch.float32, dt):
        got = torch.zeros(n, dtype=shard_dt)
        torch_ops.reduce_scatter_fanin(got, [c.clone() for c in chunks], None, False, premul=scalar)
        assert_bits_equal(got, want.to(shard_dt), "fan-in of pre-multiplied contributions vs float64")
        base = mixed_values(g, n, shard_dt, std=1e-3, specials=False)
        got = base.clone()
        torch_ops.reduce_scatter_fanin(got, [c.clone() for c in chunks], None, True, premul=scalar)
        assert_bits_equal(got, (base.double() + want.double()).float().to(shard_dt), "accumulating form")
    one = chunks[0].clone()
    torch_ops.reduce_scatter_one_rank_share(one, "PREMUL_SUM", n_src, scalar)
    alone = torch.zeros(n, dtype=dt)
    torch_ops.reduce_scatter_fanin(alone, [chunks[0].clone()], None, False, premul=scalar)
    assert_bits_equal(alone, one, "one contribution = the one-rank share")


def test_reduce_scatter_local_applies_the_collective_between_the_two_divides():
    """pre-divide (:139) on the whole buffer, the collective's share (:152-162) and the post-divide (:165) on the
    chunk, then the accumulation (:189): every step rounds to the reduce dtype."""
    g = torch.Generator().manual_seed(19)
    w, r, s = 3, 1, 1 << 12
    rs = mixed_values(g, w * s, torch.bfloat16, std=1e-3, specials=False)
    shard0 = mixed_values(g, s, torch.float32, std=1e-4, specials=False)
    shard, buf = shard0.clone(), rs.clone()
    out = torch_ops.reduce_scatter_local(shard, buf, w, r, None, None, "add", collective=("AVG", None))
    k = _scalar_in(torch.bfloat16, 1 / 3)
    chunk = (rs[r * s : (r + 1) * s].double() * k).float().to(torch.bfloat16)
    assert_bits_equal(out, chunk, "the chunk after the collective")
    assert_bits_equal(shard, (shard0.double() + chunk.double()).float(), "gradient shard")
    assert_bits_equal(buf[:s], rs[:s], "other ranks' chunks are left alone")
