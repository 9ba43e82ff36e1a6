"""The two exchange points as one-GPU kernels over several local buffers:
copy-in written to several destinations, and the reduce-scatter + post-divide
+ accumulate over several chunks; bit for bit against the torch-op oracle."""

import pytest
import torch

from oracle import torch_ops

from helpers import DTYPES, assert_bits_equal, mixed_values

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SIZES = [1, 3, 4, 1023, 2048, 100_003, (1 << 20) + 5]


@pytest.fixture(scope="module")
def nat():
    from yafsdp_amd import _native

    return _native


@pytest.mark.parametrize("src_dt", DTYPES)
@pytest.mark.parametrize("dst_dt", DTYPES)
@pytest.mark.parametrize("n_dst", [1, 3, 8, 16])
def test_copy_in_fanout(nat, src_dt, dst_dt, n_dst):
    g = torch.Generator().manual_seed(401)
    for n in SIZES:
        print("fanout", src_dt, dst_dt, n_dst, n, flush=True)
        src = mixed_values(g, n, src_dt)
        want = [torch.full((n + 8,), 7.0, dtype=dst_dt) for _ in range(n_dst)]
        torch_ops.copy_in_fanout([w[:n] for w in want], src)
        got = [torch.full((n + 8,), 7.0, dtype=dst_dt, device=DEV) for _ in range(n_dst)]
        nat.flat_copy_fanout([x[:n] for x in got], src.to(DEV))
        for k in range(n_dst):
            assert_bits_equal(got[k], want[k], f"fan-out destination {k} n={n}")


@pytest.mark.parametrize("chunk_dt,shard_dt", [(torch.bfloat16, torch.float32), (torch.float32, torch.float32),
                                               (torch.float16, torch.float32), (torch.float32, torch.bfloat16),
                                               (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("post", [None, 8.0, 3.0])
@pytest.mark.parametrize("acc", [False, True])
@pytest.mark.parametrize("n_src", [1, 2, 8, 16])
def test_reduce_fanin(nat, chunk_dt, shard_dt, post, acc, n_src):
    g = torch.Generator().manual_seed(402 + n_src)
    for n in SIZES:
        print("fanin", chunk_dt, shard_dt, post, acc, n_src, n, flush=True)
        chunks = [mixed_values(g, n, chunk_dt, 1e-3).roll(k) for k in range(n_src)]
        shard = mixed_values(g, n, shard_dt, 1e-4).flip(0)
        want = shard.clone()
        torch_ops.reduce_scatter_fanin(want, chunks, post, acc)
        got = torch.full((n + 8,), 5.0, dtype=shard_dt, device=DEV)
        got[:n] = shard.to(DEV)
        nat.post_reduce_fanin(got[:n], [c.to(DEV) for c in chunks], post, acc)
        assert_bits_equal(got[:n], want, f"fan-in n={n}")
        assert float(got[n:].float().min()) == 5.0 and float(got[n:].float().max()) == 5.0


@pytest.mark.parametrize("chunk_dt,shard_dt", [(torch.bfloat16, torch.float32), (torch.float32, torch.float32),
                                               (torch.float16, torch.float32), (torch.float32, torch.bfloat16),
                                               (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16)])
@pytest.mark.parametrize("acc", [False, True])
@pytest.mark.parametrize("n_src,scalar", [(1, 1 / 3), (3, 1 / 3), (6, 1 / 6), (8, 1 / 8), (16, 1 / 5.0), (2, 1.0)])
def test_reduce_fanin_of_a_collective_that_scales_inside_the_reduction(nat, chunk_dt, shard_dt, acc, n_src, scalar):
    """ReduceOp.AVG / the pre-multiplied sum (ya_fsdp/_collectives.py:243-249) over several ranks' chunks: each
    element times the scalar in the chunk dtype, rounded, before the binary32 sum.  Specials included: a product
    that overflows the chunk dtype becomes an infinity before the sum, as in the collective."""
    g = torch.Generator().manual_seed(404 + n_src)
    for n in SIZES:
        print("fanin premul", chunk_dt, shard_dt, acc, n_src, scalar, n, flush=True)
        chunks = [mixed_values(g, n, chunk_dt, 1e-3).roll(k) for k in range(n_src)]
        shard = mixed_values(g, n, shard_dt, 1e-4).flip(0)
        want = shard.clone()
        torch_ops.reduce_scatter_fanin(want, [c.clone() for c in chunks], None, acc, premul=scalar)
        got = torch.full((n + 8,), 5.0, dtype=shard_dt, device=DEV)
        got[:n] = shard.to(DEV)
        nat.post_reduce_fanin(got[:n], [c.to(DEV) for c in chunks], None, acc, premul=scalar)
        assert_bits_equal(got[:n], want, f"pre-multiplied fan-in n={n}")
        assert float(got[n:].float().min()) == 5.0 and float(got[n:].float().max()) == 5.0


def test_one_chunk_premultiplied_fanin_is_the_one_rank_share(nat):
    g = torch.Generator().manual_seed(405)
    n = 50_001
    chunk = mixed_values(g, n, torch.bfloat16, 1e-3).to(DEV)
    shard = mixed_values(g, n, torch.float32, 1e-4).to(DEV)
    a, b = shard.clone(), shard.clone()
    nat.post_reduce_premul(a, chunk, 1 / 3, True)
    nat.post_reduce_fanin(b, [chunk], None, True, premul=1 / 3)
    assert_bits_equal(a, b.cpu(), "single chunk, pre-multiplied")
    with pytest.raises(ValueError):
        nat.post_reduce_fanin(b, [chunk], 3.0, True, premul=1 / 3)


def test_one_chunk_fanin_is_post_reduce(nat):
    g = torch.Generator().manual_seed(403)
    n = 50_001
    chunk = mixed_values(g, n, torch.bfloat16, 1e-3).to(DEV)
    shard = mixed_values(g, n, torch.float32, 1e-4).to(DEV)
    a, b = shard.clone(), shard.clone()
    nat.post_reduce(a, chunk, 8.0, True)
    nat.post_reduce_fanin(b, [chunk], 8.0, True)
    assert_bits_equal(a, b.cpu(), "single chunk")


def test_fan_errors(nat):
    a = torch.zeros(64, device=DEV)
    with pytest.raises(ValueError):
        nat.flat_copy_fanout([], a)
    with pytest.raises(RuntimeError):
        nat.flat_copy_fanout([torch.zeros(64, device=DEV) for _ in range(17)], a)
    with pytest.raises(RuntimeError, match="aligned"):
        nat.flat_copy_fanout([torch.zeros(72, device=DEV)[1:65]], a)
    with pytest.raises(ValueError):
        nat.post_reduce_fanin(a, [torch.zeros(32, device=DEV)], None, False)
