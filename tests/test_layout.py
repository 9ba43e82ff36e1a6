"""Ragged-shard layout: closed form vs hand-derived known answers, vs the
brute-force restatement of the reference's index method, and invariants."""

import random

import pytest

from oracle.layout_bruteforce import bruteforce_layout
from yafsdp_amd._layout import RaggedShard, make_layout, padded_numel


def test_kat1_hand_derived():
    # numels=[5,3,6], W=4, A=1: T=14, T_pad=16, S=4 (rules of
    # ya_fsdp/_param_group.py:245-265 and :341-377 applied by hand)
    lay = make_layout([5, 3, 6], 4, 1)
    assert (lay.total_numel, lay.padded_unsharded_numel, lay.padded_sharded_numel) == (14, 16, 4)
    assert lay.offsets == (0, 5, 8, 14)
    expect = {
        0: ([4, 0, 0], [0, 3, 6], 0),
        1: ([1, 3, 0], [4, 0, 6], 0),
        2: ([0, 0, 4], [5, 3, 0], 0),
        3: ([0, 0, 2], [5, 3, 4], 2),
    }
    for r, (numels, offs, pad) in expect.items():
        assert lay.sharded_numels(r) == numels
        assert lay.global_offsets(r) == offs
        assert lay.pad_numel(r) == pad
    assert lay.per_rank_sharded_numels() == [(4, 1, 0, 0), (0, 3, 0, 0), (0, 0, 4, 2)]


def test_kat2_hand_derived():
    lay = make_layout([5, 3, 6], 2, 4)
    assert (lay.padded_unsharded_numel, lay.padded_sharded_numel) == (16, 8)
    assert lay.sharded_numels(0) == [5, 3, 0] and lay.global_offsets(0) == [0, 0, 6]
    assert lay.sharded_numels(1) == [0, 0, 6] and lay.global_offsets(1) == [5, 3, 0]
    assert lay.pad_numel(1) == 2
    assert lay.per_rank_sharded_numels() == [(5, 0), (3, 0), (0, 6)]


def test_placements_dataclass():
    lay = make_layout([5, 3, 6], 4, 1)
    pl = lay.placements(1)
    assert pl[0] == RaggedShard(1, 4, (4, 1, 0, 0))
    assert str(pl[1]) == "RS(3, 0)"


LLAMA8B = [4096 * 4096, 1024 * 4096, 1024 * 4096, 4096 * 4096, 14336 * 4096, 14336 * 4096, 4096 * 14336, 4096, 4096]
LLAMA70B = [8192 * 8192, 1024 * 8192, 1024 * 8192, 8192 * 8192, 28672 * 8192, 28672 * 8192, 8192 * 28672, 8192, 8192]


def test_llama8b_layer_w8():
    for a in (8, 512):
        lay = make_layout(LLAMA8B, 8, a)
        assert lay.total_numel == lay.padded_unsharded_numel == 218_112_000
        assert lay.padded_sharded_numel == 27_264_000
    lay = make_layout(LLAMA8B, 8, 512)
    assert lay.sharded_numels(0) == [16_777_216, 4_194_304, 4_194_304, 2_098_176, 0, 0, 0, 0, 0]
    n1 = lay.sharded_numels(1)
    assert n1[3] == 14_679_040 and n1[4] == 12_584_960 and lay.global_offsets(1)[3] == 2_098_176
    n3 = lay.sharded_numels(3)
    assert n3[4] == 18_871_296 and n3[5] == 8_392_704 and lay.global_offsets(3)[4] == 39_848_960
    n7 = lay.sharded_numels(7)
    assert n7[6:] == [27_255_808, 4096, 4096] and lay.global_offsets(7)[6] == 31_464_448


def test_llama70b_layer_w64():
    lay8 = make_layout(LLAMA70B, 64, 8)
    assert lay8.total_numel == 855_654_400 == lay8.padded_unsharded_numel
    assert lay8.padded_sharded_numel == 13_369_600
    lay = make_layout(LLAMA70B, 64, 512)
    assert lay.padded_unsharded_numel == 855_670_784 and lay.padded_sharded_numel == 13_369_856
    last = lay.sharded_numels(63)
    assert last[6:] == [13_337_088, 8192, 8192] and lay.pad_numel(63) == 16_384
    assert lay.global_offsets(63)[6] == 221_543_936
    # ranks 0 and 1 lie wholly inside q
    for r in (0, 1):
        assert lay.sharded_numels(r)[0] == lay.padded_sharded_numel


@pytest.mark.parametrize("seed", range(60))
def test_closed_form_vs_bruteforce(seed):
    rng = random.Random(seed)
    p = rng.randint(1, 8)
    numels = [rng.randint(0 if rng.random() < 0.1 else 1, 50) for _ in range(p)]
    if sum(numels) == 0:
        numels[0] = 1
    w = rng.randint(1, 7)
    a = rng.choice([1, 2, 3, 4, 8])
    lay = make_layout(numels, w, a)
    for r in range(w):
        bf = bruteforce_layout(numels, w, a, r)
        assert lay.total_numel == bf["total"]
        assert lay.padded_unsharded_numel == bf["padded"]
        assert lay.padded_sharded_numel == bf["shard"]
        assert lay.sharded_numels(r) == bf["sharded_numels"]
        assert lay.global_offsets(r) == bf["global_offsets"]
        assert lay.per_rank_sharded_numels() == bf["per_rank_sharded_numels"]


@pytest.mark.parametrize("seed", range(20))
def test_invariants_large(seed):
    rng = random.Random(1000 + seed)
    p = rng.randint(1, 300)
    numels = [int(2 ** rng.uniform(0, 22)) | 1 for _ in range(p)]
    w = rng.choice([1, 2, 8, 64, 256])
    a = rng.choice([1, 8, 512])
    lay = make_layout(numels, w, a)
    s = lay.padded_sharded_numel
    assert lay.padded_unsharded_numel % (w * a) == 0
    assert 0 <= lay.padded_unsharded_numel - lay.total_numel < w * a
    per_rank = lay.per_rank_sharded_numels()
    for pi, n in enumerate(numels):
        assert sum(per_rank[pi]) == n
    tot_pad = 0
    for r in range(w):
        sn = lay.sharded_numels(r)
        assert sum(sn) + lay.pad_numel(r) == s
        assert [per_rank[pi][r] for pi in range(p)] == sn
        tot_pad += lay.pad_numel(r)
        go = lay.global_offsets(r)
        for pi, n in enumerate(numels):
            if sn[pi] > 0:
                assert lay.offsets[pi] + go[pi] >= r * s
                assert lay.offsets[pi] + go[pi] + sn[pi] <= (r + 1) * s
            else:
                assert go[pi] == n
    assert tot_pad == lay.padded_unsharded_numel - lay.total_numel


def test_padded_numel_and_errors():
    assert padded_numel(14, 4, 1) == 16
    assert padded_numel(16, 4, 1) == 16
    assert padded_numel(1, 256, 512) == 256 * 512
    with pytest.raises(ValueError):
        make_layout([1], 0, 8)
    with pytest.raises(ValueError):
        make_layout([1], 2, 8).sharded_numels(2)
    with pytest.raises(AssertionError):
        make_layout([1] * 65535, 2, 8)
