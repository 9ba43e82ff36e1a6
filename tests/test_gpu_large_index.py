"""Buffers of more than 2^31 elements: every index on the path is 64-bit.  At
this size the checks are size-independent properties (byte identity of copies,
exact power-of-two scaling, a sum whose value is known in closed form), computed
on the GPU with torch ops on the same device buffers."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
N = (1 << 31) + 12_345  # elements


@pytest.fixture(scope="module")
def nat():
    from yafsdp_amd import _native

    return _native


@pytest.fixture(scope="module")
def pattern():
    """bf16 values +-2^k, k in [-7, 8): exact under scaling by powers of two, squares exactly representable."""
    idx = torch.arange(N, device=DEV, dtype=torch.int64)
    expo = (idx % 15 - 7).to(torch.float32)
    sign = 1.0 - 2.0 * ((idx // 15) % 2).to(torch.float32)
    x = (sign * torch.exp2(expo)).to(torch.bfloat16)
    del idx, expo, sign
    return x


def test_flat_copy_fill_and_sumsq_beyond_int32(nat, pattern):
    print("flat ops on", N, "elements", flush=True)
    dst = torch.empty(N, dtype=torch.bfloat16, device=DEV)
    nat.flat_copy(dst, pattern)
    assert torch.equal(dst.view(torch.int16), pattern.view(torch.int16))
    # sum of squares: every window of 15 elements adds up to sum_k 4^k, k = -7..7
    out = torch.zeros(1, dtype=torch.float64, device=DEV)
    nat.flat_sumsq(pattern, out, nat.sumsq_workspace(DEV))
    full, rest = divmod(N, 15)
    want = full * sum(4.0**k for k in range(-7, 8)) + sum(4.0**k for k in range(-7, -7 + rest))
    assert out.item() == want, (out.item(), want)
    nat.flat_fill(dst, -0.5)
    assert int((dst.view(torch.int16) != torch.tensor(-0.5, dtype=torch.bfloat16).view(torch.int16).item()).sum()) == 0
    del dst


def test_table_with_offsets_beyond_int32(nat, pattern):
    """Two tensors, the second starting beyond element 2^31 of the flat buffer: reduce copy-in with /8 into a
    bf16 buffer and copy-out back, both exact."""
    n0 = (1 << 31) + 5
    numels = [n0, N - n0]
    padded = N + 27
    print("table ops, offsets", [0, n0], flush=True)
    table = nat.TensorTable(numels, padded, DEV)
    flat = torch.full((padded,), 3.0, dtype=torch.bfloat16, device=DEV)
    table.gather_in([pattern[:n0], pattern[n0:]], flat, None, 8.0, True)
    for lo, hi in ((0, 1 << 20), (n0 - (1 << 20), N)):  # the start, and the seam up to the end
        want = (pattern[lo:hi].float() / 8.0).to(torch.bfloat16)
        assert torch.equal(flat[lo:hi].view(torch.int16), want.view(torch.int16)), (lo, hi)
    # whole buffer through an exact checksum: scaling by 1/8 is exact, so sum(|flat|) * 8 == sum(|pattern|)
    assert flat[:N].float().abs().sum(dtype=torch.float64).item() * 8.0 == pattern.float().abs().sum(dtype=torch.float64).item()
    assert float(flat[N:].float().abs().max()) == 0.0  # pad lanes zero-filled
    outs = [torch.empty(n, dtype=torch.bfloat16, device=DEV) for n in numels]
    table.scatter_out(flat, outs)
    assert torch.equal(outs[0].view(torch.int16), flat[:n0].view(torch.int16))
    assert torch.equal(outs[1].view(torch.int16), flat[n0:N].view(torch.int16))
    table.close()


def test_shared_launches_beyond_int32(nat, pattern):
    """The two launches that do the work of two each on the same table: copy-in + copy-out as one grid, and the
    one-pass reduce of a size-one group (with a /4 before and a /2 after the reduce buffer, both exact here)."""
    n0 = (1 << 31) + 5
    numels = [n0, N - n0]
    padded = N + 27
    print("shared launches, offsets", [0, n0], flush=True)
    table = nat.TensorTable(numels, padded, DEV)
    # copy-in + copy-out
    gathered = torch.empty(padded, dtype=torch.bfloat16, device=DEV)
    gathered[:N].copy_(pattern)
    gathered[N:].fill_(7.0)
    master = pattern[: 1 << 22].float() * 3.0
    ag = torch.zeros(1 << 22, dtype=torch.bfloat16, device=DEV)
    outs = [torch.empty(n, dtype=torch.bfloat16, device=DEV) for n in numels]
    assert table.copy_in_scatter_out(gathered, outs, ag, master)
    assert torch.equal(ag.view(torch.int16), master.to(torch.bfloat16).view(torch.int16))
    assert torch.equal(outs[0].view(torch.int16), pattern[:n0].view(torch.int16))
    assert torch.equal(outs[1].view(torch.int16), pattern[n0:].view(torch.int16))
    del gathered, outs, ag, master
    # one-pass reduce: flat = pattern / 4 (pad zero), shard = 1.0 + flat / 2 in binary32 (all exact)
    flat = torch.full((padded,), 3.0, dtype=torch.bfloat16, device=DEV)
    shard = torch.ones(padded, dtype=torch.float32, device=DEV)
    assert table.gather_in_post_reduce([pattern[:n0], pattern[n0:]], flat, shard, True, pre_factor=4.0, post_factor=2.0)
    for lo, hi in ((0, 1 << 20), (n0 - (1 << 20), N)):
        want = (pattern[lo:hi].float() / 4.0).to(torch.bfloat16)
        assert torch.equal(flat[lo:hi].view(torch.int16), want.view(torch.int16)), (lo, hi)
        assert torch.equal(shard[lo:hi], 1.0 + want.float() / 2.0), (lo, hi)
    assert flat[:N].float().abs().sum(dtype=torch.float64).item() * 4.0 == pattern.float().abs().sum(dtype=torch.float64).item()
    assert float(flat[N:].float().abs().max()) == 0.0 and float((shard[N:] - 1.0).abs().max()) == 0.0
    # the whole shard through an exact checksum: sum(shard - 1) * 8 == sum(pattern) (every term a small power of two)
    got = (shard[:N] - 1.0).sum(dtype=torch.float64).item() * 8.0
    assert got == pattern.float().sum(dtype=torch.float64).item(), got
    table.close()
