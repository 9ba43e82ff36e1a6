"""Closed-form ragged-shard layout of one parameter group's flat buffer.

The reference derives the same quantities by materialising one uint16 parameter
index and one int64 element index per element of the padded buffer and counting
matches per (parameter, rank) with device->host syncs
(ya_fsdp/_param_group.py:284-377).  Everything it computes is an interval
intersection, so this module does it with integer arithmetic on the host:

* sizing (ya_fsdp/_param_group.py:245-265):
      T      = sum(numels)
      T_pad  = T rounded up to a multiple of W * shard_alignment
      S      = T_pad // W
* parameter p occupies the flat range [o_p, o_p + N_p); rank r owns
  [r*S, (r+1)*S).  ``sharded_numel[p]`` is the length of the intersection and
  ``global_offset[p]`` is the first element of p the rank holds, or N_p when it
  holds none (ya_fsdp/_param_group.py:359-377).
* ``shard_numels[p]`` lists the intersection lengths for ranks 0..W-1
  (ya_fsdp/_param_group.py:347-353, consumed by RaggedShard at
  ya_fsdp/_tensor.py:41-51).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from itertools import accumulate
from typing import Sequence

# ya_fsdp/_param_group.py:284-287 keeps one uint16 index per element and asserts
# len(params) < 65535; the limit is kept so a group valid here is valid there.
MAX_PARAMS_PER_GROUP = 65535


@dataclass(frozen=True)
class RaggedShard:
    """Placement of one parameter on one rank (ya_fsdp/_tensor.py:41-51)."""

    local_numel: int
    global_offset: int
    shard_numels: tuple[int, ...]

    def __repr__(self) -> str:
        return (
            f"RaggedShard(local_numel={self.local_numel}, "
            f"global_offset={self.global_offset})"
        )

    def __str__(self) -> str:
        return f"RS({self.local_numel}, {self.global_offset})"


def padded_numel(total_numel: int, world_size: int, shard_alignment: int) -> int:
    """T_pad: ``total_numel`` rounded up to ``world_size * shard_alignment``
    (ya_fsdp/_param_group.py:252-257)."""
    divider = world_size * shard_alignment
    rem = total_numel % divider
    return total_numel if rem == 0 else total_numel + (divider - rem)


@dataclass(frozen=True)
class ShardLayout:
    """Layout of one (group, all-gather dtype) flat buffer for every rank."""

    numels: tuple[int, ...]
    world_size: int
    shard_alignment: int
    # derived
    offsets: tuple[int, ...] = field(init=False)  # P+1 prefix offsets, offsets[P] == T
    total_numel: int = field(init=False)  # T
    padded_unsharded_numel: int = field(init=False)  # T_pad
    padded_sharded_numel: int = field(init=False)  # S

    def __post_init__(self) -> None:
        if self.world_size < 1:
            raise ValueError(f"world_size must be >= 1, got {self.world_size}")
        if self.shard_alignment < 1:
            raise ValueError(f"shard_alignment must be >= 1, got {self.shard_alignment}")
        if any(n < 0 for n in self.numels):
            raise ValueError("parameter numels must be non-negative")
        if len(self.numels) >= MAX_PARAMS_PER_GROUP:
            raise AssertionError(
                f"a group holds fewer than {MAX_PARAMS_PER_GROUP} parameters, got {len(self.numels)}"
            )
        offsets = (0, *accumulate(self.numels))
        object.__setattr__(self, "numels", tuple(int(n) for n in self.numels))
        object.__setattr__(self, "offsets", tuple(offsets))
        object.__setattr__(self, "total_numel", offsets[-1])
        t_pad = padded_numel(offsets[-1], self.world_size, self.shard_alignment)
        object.__setattr__(self, "padded_unsharded_numel", t_pad)
        object.__setattr__(self, "padded_sharded_numel", t_pad // self.world_size)

    # ---- per-rank quantities -------------------------------------------------
    def rank_range(self, rank: int) -> tuple[int, int]:
        """Flat range [lo, hi) of the padded buffer owned by ``rank``
        (``torch.chunk(buffer, W)[rank]`` on a length divisible by W)."""
        self._check_rank(rank)
        s = self.padded_sharded_numel
        return rank * s, (rank + 1) * s

    def sharded_numels(self, rank: int) -> list[int]:
        """``sharded_param_numels`` of ya_fsdp/_param_group.py:354-358."""
        lo, hi = self.rank_range(rank)
        return [
            max(0, min(hi, self.offsets[p + 1]) - max(lo, self.offsets[p]))
            for p in range(len(self.numels))
        ]

    def global_offsets(self, rank: int) -> list[int]:
        """``sharded_data_global_offsets`` of ya_fsdp/_param_group.py:359-377:
        smallest element index of p present on the rank, N_p if none is."""
        lo, hi = self.rank_range(rank)
        out = []
        for p, n in enumerate(self.numels):
            a, b = max(lo, self.offsets[p]), min(hi, self.offsets[p + 1])
            out.append(a - self.offsets[p] if b > a else n)
        return out

    def per_rank_sharded_numels(self) -> list[tuple[int, ...]]:
        """``per_rank_sharded_param_numels`` (ya_fsdp/_param_group.py:347-353):
        for every parameter, its element count on ranks 0..W-1."""
        s = self.padded_sharded_numel
        out = []
        for p, n in enumerate(self.numels):
            row = [0] * self.world_size
            if n > 0 and s > 0:
                o = self.offsets[p]
                first, last = o // s, (o + n - 1) // s
                for r in range(first, last + 1):
                    row[r] = min((r + 1) * s, o + n) - max(r * s, o)
            out.append(tuple(row))
        return out

    def placements(self, rank: int) -> list[RaggedShard]:
        """One RaggedShard per parameter, as built at ya_fsdp/_param.py:96-103."""
        per_rank = self.per_rank_sharded_numels()
        return [
            RaggedShard(local_numel=ln, global_offset=go, shard_numels=sn)
            for ln, go, sn in zip(
                self.sharded_numels(rank), self.global_offsets(rank), per_rank
            )
        ]

    def pad_numel(self, rank: int) -> int:
        """Number of pad lanes (beyond T) inside the rank's shard."""
        lo, hi = self.rank_range(rank)
        return max(0, hi - max(lo, self.total_numel))

    def _check_rank(self, rank: int) -> None:
        if not 0 <= rank < self.world_size:
            raise ValueError(f"rank {rank} outside [0, {self.world_size})")


def make_layout(
    numels: Sequence[int], world_size: int, shard_alignment: int = 8
) -> ShardLayout:
    """``shard_alignment`` defaults to 8 elements as in ya_fsdp/fully_shard.py:75."""
    return ShardLayout(tuple(numels), int(world_size), int(shard_alignment))
