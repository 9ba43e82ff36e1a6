"""Shard-group description and training states.

The reference takes its shard world size and rank from a ``DeviceMesh`` and a
``ProcessGroup`` (ya_fsdp/_common.py:13-35).  This build runs on one GPU: the
world size is a layout parameter, so the group is a plain ``(size, rank)``
pair with the two methods of ``ProcessGroup`` the buffer path calls.
"""

from __future__ import annotations

import contextlib
from dataclasses import dataclass
from enum import Enum, auto

import torch


class LogicalShardGroup:
    """Stands where ``dist.ProcessGroup`` stands in ya_fsdp/_collectives.py:
    ``size()`` and ``rank()`` are all the path reads from it.  No inter-GPU
    exchange is attached: with ``size() > 1`` the all-gather fills only this
    rank's slot of the gathered buffer and the reduce-scatter result is this
    rank's chunk of the reduce buffer (peers contribute nothing)."""

    def __init__(self, size: int, rank: int):
        if size < 1 or not 0 <= rank < size:
            raise ValueError(f"invalid shard group: size={size} rank={rank}")
        self._size, self._rank = int(size), int(rank)

    def size(self) -> int:
        return self._size

    def rank(self) -> int:
        return self._rank

    def __repr__(self) -> str:
        return f"LogicalShardGroup(size={self._size}, rank={self._rank})"

    # two logical groups of equal size and rank are the same group (every fully_shard call builds its own
    # object), so dictionaries keyed by "the process group" work as they do with real process groups
    def __eq__(self, other: object) -> bool:
        return isinstance(other, LogicalShardGroup) and (self._size, self._rank) == (other._size, other._rank)

    def __hash__(self) -> int:
        return hash((LogicalShardGroup, self._size, self._rank))


@dataclass
class FSDPMeshInfo:
    """``shard_mesh_size`` / ``shard_mesh_rank`` / ``shard_process_group`` as in
    ya_fsdp/_common.py:25-34, built from the two integers instead of a mesh."""

    shard_mesh_size: int
    shard_mesh_rank: int

    def __post_init__(self) -> None:
        self.shard_process_group = LogicalShardGroup(self.shard_mesh_size, self.shard_mesh_rank)


class TrainingState(Enum):
    """ya_fsdp/_common.py:37-45."""

    FORWARD = auto()
    PRE_BACKWARD = auto()
    POST_BACKWARD = auto()
    IDLE = auto()


class ShardedState(Enum):
    """ya_fsdp/_param.py:33-41 without the post-forward state (no HSDP here)."""

    SHARDED = auto()
    UNSHARDED = auto()


def resolve_device(device: "torch.device | str | int | None") -> torch.device:
    """A device with an explicit index: ``"cuda"`` means the current GPU, as the reference's device handle
    resolves it (ya_fsdp/fully_shard.py:110-113 through ``_get_device_from_mesh``).  Tensors always report an
    indexed device, so comparisons against ``cuda`` without an index would never match."""
    device = torch.device(f"cuda:{torch.cuda.current_device()}" if device is None else device)
    if device.type == "cuda" and device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    return device


def is_bw() -> bool:
    """ya_fsdp/_common.py:73-74."""
    return torch._C._current_graph_task_id() != -1


_NO_RANGE = contextlib.nullcontext()


def profiler_range(name: str):
    """``torch.profiler.record_function(name)`` while a torch profiler (or an NVTX / ITT emitter) is running, a
    shared no-op context otherwise: the ranges the reference opens around every hook cost about 7 us each on the
    host when nobody records them."""
    if torch.autograd.profiler._is_profiler_enabled:
        return torch.profiler.record_function(name)
    return _NO_RANGE
