"""Chunk metadata of the sharded checkpoint format (ya_fsdp/_tensor.py:365-423)
from the closed-form layout, against hand-derived known answers."""

from yafsdp_amd._layout import make_layout
from yafsdp_amd.checkpoint import chunk_meta


def test_known_answer_three_params_four_ranks():
    # numels [5, 3, 6], W = 4, alignment 1: T_pad = 16, S = 4
    lay = make_layout([5, 3, 6], 4, 1)
    shapes = [(5,), (3, 1), (2, 3)]
    want = {
        0: [((0,), (4,)), ((3,), (0,)), ((6,), (0,))],
        1: [((4,), (1,)), ((0,), (3,)), ((6,), (0,))],
        2: [((5,), (0,)), ((3,), (0,)), ((0,), (4,))],
        3: [((5,), (0,)), ((3,), (0,)), ((4,), (2,))],
    }
    for rank, expected in want.items():
        metas = [chunk_meta(f"p{i}", pl, shapes[i]) for i, pl in enumerate(lay.placements(rank))]
        assert [(m.offsets, m.sizes) for m in metas] == expected, rank
        assert [m.size for m in metas] == [(5,), (3,), (6,)]
        assert [m.shape for m in metas] == [(5,), (3, 1), (2, 3)]


def test_chunks_of_all_ranks_tile_every_parameter():
    numels = [7, 1, 130, 64, 3]
    for w, a in ((1, 8), (3, 8), (5, 1), (8, 2)):
        lay = make_layout(numels, w, a)
        for p, n in enumerate(numels):
            pos = 0
            for r in range(w):
                m = chunk_meta("x", lay.placements(r)[p], (n,))
                if m.sizes[0]:
                    assert m.offsets[0] == pos  # chunks follow one another in rank order
                    pos += m.sizes[0]
                else:
                    assert m.offsets == (n,)
            assert pos == n
