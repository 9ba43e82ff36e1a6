"""Sharded checkpoint format of the ragged shards, and conversion to and from
full parameters on one GPU.

In the reference a sharded parameter is saved as ONE chunk of the parameter
flattened to 1-D: ``offsets = (global_offset,)`` (or ``(numel,)`` when the rank
holds nothing of it), ``sizes = (local_numel,)``, full ``size = (numel,)``
(``__create_write_items__`` / ``__create_chunk_list__``,
ya_fsdp/_tensor.py:365-423), and ``full_tensor()`` is an all-gather of the
local tensors into ``full.split(shard_numels)`` (ya_fsdp/_tensor.py:345-363).
The legacy wrapper stores names, element counts and shapes per module next to
its flat shards (``_meta_info``, ya_fsdp/ya_fsdp.py:236-245).

Here the same metadata comes from the closed-form layout, and the byte
movement runs on the buffer kernels: the ranks' flat shards are copied into a
flat buffer (``flat_copy``) and split into the full parameters by the copy-out
kernel (``scatter_out``); loading copies each rank's fragment out of the full
parameter (``flat_copy``).  One GPU: the "ranks" are the logical ranks of a
layout, e.g. modules wrapped with ``mesh=(W, r)``.  ``RaggedShardTensor`` hands the
same chunks to ``torch.distributed.checkpoint`` (the hooks of
ya_fsdp/_tensor.py:365-432).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, Mapping, Sequence

import torch
import torch.nn as nn

from . import _native
from ._layout import RaggedShard
from ._param_group import YaFSDPParamGroup

__all__ = ["ChunkMeta", "chunk_meta", "sharded_state_dict", "group_meta_info", "full_tensors", "load_full_tensors",
           "full_state_dict", "load_full_state_dict", "RaggedShardTensor", "checkpointable_state_dict",
           "RaggedShardLoadPlanner"]


@dataclass(frozen=True)
class ChunkMeta:
    """What the reference writes for one sharded parameter on one rank."""

    fqn: str
    offsets: tuple[int, ...]  # position of the chunk in the flattened parameter
    sizes: tuple[int, ...]  # its length
    size: tuple[int, ...]  # the flattened parameter's size
    shape: tuple[int, ...]  # the parameter's original shape


def chunk_meta(fqn: str, placement: RaggedShard, shape: Sequence[int]) -> ChunkMeta:
    """ya_fsdp/_tensor.py:365-392 for a 1-D shard mesh: an empty fragment is
    placed at ``offset == numel`` (its ``global_offset`` already is,
    ya_fsdp/_param_group.py:365-377)."""
    numel = 1
    for d in shape:
        numel *= int(d)
    if placement.local_numel == 0:
        offsets = (numel,)
    else:
        offsets = (placement.global_offset,)
    return ChunkMeta(fqn, offsets, (placement.local_numel,), (numel,), tuple(int(d) for d in shape))


def sharded_state_dict(group: YaFSDPParamGroup) -> dict[str, tuple[torch.Tensor, ChunkMeta]]:
    """``{fqn: (local 1-D tensor, chunk)}`` of one parameter group on this rank;
    the tensors are views of the flat master shard (no copy)."""
    out = {}
    for fsdp_param in group.fsdp_params:
        meta = chunk_meta(fsdp_param._param_fqn, fsdp_param.placement, fsdp_param._orig_size)
        out[fsdp_param._param_fqn] = (fsdp_param._sharded_param_data, meta)
    return out


class RaggedShardTensor(torch.Tensor):
    """Checkpoint handle of one parameter on one rank: stands for the parameter
    flattened to ``(numel,)`` (that is its ``size()``; it has no storage of its
    own) and holds the rank's local 1-D fragment, with the three hooks that
    ``torch.distributed.checkpoint`` looks for on a state-dict value
    (``__create_write_items__``, ``__create_chunk_list__``, ``__get_tensor_shard__``)
    and the chunk the reference declares (ya_fsdp/_tensor.py:365-432): this
    rank contributes ``[offset, offset + local_numel)`` of the flattened
    parameter, or an empty chunk at ``offset == numel``.  The local fragment
    aliases the tensor given (normally a view of the flat master shard), so
    saving reads the masters and loading writes them; after a load, clear the
    group's copy-in flags (``load_full_tensors`` shows how) so that the next
    unshard casts the new values.  No tensor op runs on the handle itself."""

    __slots__ = ["_local_tensor", "_chunk"]

    @staticmethod
    def __new__(cls, local: torch.Tensor, meta: ChunkMeta) -> "RaggedShardTensor":
        if local.dim() != 1 or local.numel() != meta.sizes[0]:
            raise ValueError(f"{meta.fqn}: local tensor {tuple(local.shape)} does not match the chunk size {meta.sizes}")
        r = torch.Tensor._make_wrapper_subclass(
            cls, torch.Size(meta.size), dtype=local.dtype, device=local.device, layout=local.layout, requires_grad=False
        )
        r._local_tensor = local.detach()
        r._chunk = meta
        return r

    @classmethod
    def wrap(cls, local: torch.Tensor, meta: ChunkMeta) -> "RaggedShardTensor":
        return cls(local, meta)

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        raise NotImplementedError(f"{func}: a RaggedShardTensor is a checkpoint handle; operate on .local_tensor")

    def __repr__(self) -> str:  # type: ignore[override]
        return f"RaggedShardTensor({self._chunk}, local_tensor={self._local_tensor!r})"

    @property
    def chunk(self) -> ChunkMeta:
        return self._chunk

    @property
    def local_tensor(self) -> torch.Tensor:
        return self._local_tensor

    def _local(self) -> torch.Tensor:
        return self._local_tensor

    def __create_write_items__(self, fqn: str, object):  # noqa: A002  (the protocol's argument name)
        from torch.distributed.checkpoint.metadata import ChunkStorageMetadata, MetadataIndex, TensorProperties
        from torch.distributed.checkpoint.planner import TensorWriteData, WriteItem, WriteItemType

        offsets, sizes = torch.Size(self._chunk.offsets), torch.Size(self._chunk.sizes)
        return [
            WriteItem(
                index=MetadataIndex(fqn, offsets),
                type=WriteItemType.SHARD,
                tensor_data=TensorWriteData(
                    chunk=ChunkStorageMetadata(offsets=offsets, sizes=sizes),
                    properties=TensorProperties.create_from_tensor(self._local()),
                    size=torch.Size(self._chunk.size),
                ),
            )
        ]

    def __create_chunk_list__(self):
        from torch.distributed.checkpoint.metadata import ChunkStorageMetadata

        return [ChunkStorageMetadata(offsets=torch.Size(self._chunk.offsets), sizes=torch.Size(self._chunk.sizes))]

    def __get_tensor_shard__(self, index) -> torch.Tensor:
        return self._local()


def checkpointable_state_dict(group: YaFSDPParamGroup) -> dict[str, torch.Tensor]:
    """``{fqn: sharded parameter}`` of one parameter group on this rank, for
    ``torch.distributed.checkpoint.save`` / ``load``: the group's own
    ``RaggedShardDTensor`` parameters (detached; their local fragments are views
    of the flat master shard, so nothing is copied), which carry the checkpoint
    hooks themselves.  ``module.state_dict()`` of a ``fully_shard`` module holds
    the same tensors under the module's own names."""
    return {fsdp_param._param_fqn: fsdp_param.sharded_param.detach() for fsdp_param in group.fsdp_params}


class _FlattenedView:
    """What the load planner looks at in place of a sharded parameter: the flattened size the chunk format
    declares, and the parameter's own chunk list."""

    def __init__(self, tensor: torch.Tensor):
        self._tensor = tensor

    def size(self) -> torch.Size:
        return torch.Size((self._tensor.numel(),))

    def __create_chunk_list__(self):
        return self._tensor.__create_chunk_list__()


def _load_planner_base():
    from torch.distributed.checkpoint.default_planner import DefaultLoadPlanner

    return DefaultLoadPlanner


class RaggedShardLoadPlanner(_load_planner_base()):  # type: ignore[misc]
    """``torch.distributed.checkpoint.load(module.state_dict(), ..., planner=RaggedShardLoadPlanner())``.

    The chunk format of a ragged shard (ya_fsdp/_tensor.py:365-423) declares the parameter FLATTENED:
    ``size = (numel,)`` with 1-D offsets and lengths, while the sharded parameter itself reports the parameter's
    original shape.  The default load planner of the installed torch compares the two sizes before it plans
    anything and refuses; this planner shows it the flattened size for ``RaggedShardDTensor`` values and leaves
    everything else to the default (saving needs no planner).  Loaded values land in the local fragments, i.e.
    in the flat master shards."""

    def create_local_plan(self):
        from ._tensor import RaggedShardDTensor

        real = self.state_dict
        self.state_dict = {k: _FlattenedView(v) if isinstance(v, RaggedShardDTensor) else v for k, v in real.items()}
        try:
            return super().create_local_plan()
        finally:
            self.state_dict = real


def _one_class(group: YaFSDPParamGroup) -> None:
    if group.has_extension_classes:
        raise NotImplementedError(
            f"{group} has tensor-subclass all-gather dtype classes (all_gather_dtype_to_param_cls), each with a flat "
            "shard of its own: the legacy per-group record describes one flat buffer; full_tensors, "
            "sharded_state_dict, full_state_dict and the sharded parameters' own checkpoint hooks serve every class"
        )


def group_meta_info(group: YaFSDPParamGroup) -> dict[str, list]:
    """The per-module record the legacy wrapper keeps in its state dict
    (ya_fsdp/ya_fsdp.py:236-245), for one group."""
    _one_class(group)
    return {
        "shard_boundaries": list(group.layout.rank_range(group.mesh_info.shard_mesh_rank)),
        "padded_numel": group.layout.padded_unsharded_numel,
        "fqns": [p._param_fqn for p in group.fsdp_params],
        "numels": [p._orig_size.numel() for p in group.fsdp_params],
        "orig_shapes": [tuple(p._orig_size) for p in group.fsdp_params],
    }


def _check_ranks(groups: Sequence[YaFSDPParamGroup]) -> None:
    w = groups[0].mesh_info.shard_mesh_size
    if len(groups) != w:
        raise ValueError(f"need the groups of all {w} ranks, got {len(groups)}")
    for r, g in enumerate(groups):
        if g.layouts != groups[0].layouts or g.mesh_info.shard_mesh_rank != r:
            raise ValueError("groups must be the same parameter group on ranks 0..W-1, in rank order")


def full_tensors(
    rank_groups: Sequence[YaFSDPParamGroup], out: Mapping[str, torch.Tensor] | None = None
) -> dict[str, torch.Tensor]:
    """``full_tensor()`` of every parameter of a group (ya_fsdp/_tensor.py:345-363)
    from the flat master shards of all its ranks: per all-gather dtype class of
    the group W ``flat_copy`` launches into a flat buffer and one ``scatter_out``
    launch into the full parameters (plain tensors of the master values, also
    for tensor-subclass parameters).  ``out`` may provide destination tensors
    (master dtype, contiguous) by fqn."""
    _check_ranks(rank_groups)
    g0 = rank_groups[0]
    dtype, device = g0.orig_dtype, g0.device
    result = {}
    for key, fsdp_params in g0._all_gather_dtype_to_fsdp_params.items():
        lay = g0.layouts[key]
        s = lay.padded_sharded_numel
        flat = torch.empty(lay.padded_unsharded_numel, dtype=dtype, device=device)
        for r, g in enumerate(rank_groups):
            _native.flat_copy(flat[r * s : (r + 1) * s], g._padded_sharded_param_data[key])
        dsts = []
        for fsdp_param in fsdp_params:
            fqn = fsdp_param._param_fqn
            t = out[fqn] if out is not None and fqn in out else torch.empty(fsdp_param._orig_size, dtype=dtype, device=device)
            if t.dtype != dtype or tuple(t.shape) != tuple(fsdp_param._orig_size) or not t.is_contiguous():
                raise ValueError(f"{fqn}: destination must be a contiguous {dtype} tensor of shape {tuple(fsdp_param._orig_size)}")
            result[fqn] = t
            dsts.append(t.view(-1))
        table = _native.TensorTable([d.numel() for d in dsts], lay.padded_unsharded_numel, device)
        try:
            table.scatter_out(flat, dsts)
        finally:
            table.close()
    # in the group's parameter order, whatever the classes
    return {p._param_fqn: result[p._param_fqn] for p in g0.fsdp_params}


def load_full_tensors(groups: YaFSDPParamGroup | Iterable[YaFSDPParamGroup], full: Mapping[str, torch.Tensor]) -> None:
    """The reverse: each given group (one rank of it, or several) takes its
    fragment ``full[fqn].view(-1)[offset : offset + size]`` of every parameter
    (the chunk of ``chunk_meta``), cast to the master dtype.  Runs on the
    current stream; the next unshard casts the new masters (the group's
    once-per-iteration copy-in flag is cleared)."""
    if isinstance(groups, YaFSDPParamGroup):
        groups = [groups]
    for group in groups:
        for fsdp_param in group.fsdp_params:
            fqn = fsdp_param._param_fqn
            if fqn not in full:
                raise KeyError(f"{fqn} is missing from the full state dict")
            src = full[fqn]
            if src.numel() != fsdp_param._orig_size.numel():
                raise ValueError(f"{fqn}: expected {fsdp_param._orig_size.numel()} elements, got {src.numel()}")
            n = fsdp_param.placement.local_numel
            if n == 0:
                continue
            go = fsdp_param.placement.global_offset
            src = src.detach().to(group.device).contiguous().view(-1)
            _native.flat_copy(fsdp_param._sharded_param_data, src[go : go + n])
        group._all_gather_input_set_dtypes.clear()
        group._copy_in_shard_version = None


def fsdp_groups_of(module: nn.Module) -> list[YaFSDPParamGroup]:
    """Parameter groups of every ``fully_shard`` module under ``module``."""
    from .optim import fsdp_param_groups

    return fsdp_param_groups(module)


def _owners_by_name(module: nn.Module) -> dict[str, object]:
    """``{root-relative parameter name: owning YaFSDPParam or the plain parameter}`` of a module whose
    ``fully_shard`` groups are all in the sharded state."""
    out = {}
    for name, p in module.named_parameters(remove_duplicate=False):
        ref = getattr(p, "_yafsdp_param", None)
        owner = ref() if ref is not None else None
        if owner is not None and owner.sharded_param is not p:
            raise RuntimeError(f"{name} is not in the sharded state; call reshard() on its module first")
        out[name] = owner if owner is not None else p
    return out


def full_state_dict(module: nn.Module) -> dict[str, torch.Tensor]:
    """Parameters in their original shapes and master dtype (copies) plus buffers, for a module whose
    groups all have world size 1 (one GPU holds every parameter whole): the ordinary ``state_dict`` of the
    unwrapped model.  Larger logical world sizes go through ``full_tensors`` with the groups of all ranks."""
    out: dict[str, torch.Tensor] = {}
    for name, owner in _owners_by_name(module).items():
        if isinstance(owner, torch.Tensor):
            out[name] = owner.detach().clone()
            continue
        if owner.mesh_info.shard_mesh_size != 1:
            raise ValueError(f"{name} is sharded over {owner.mesh_info.shard_mesh_size} logical ranks; use full_tensors")
        out[name] = owner._sharded_param_data.detach().view(owner._orig_size).clone()
    for name, b in _persistent_buffers(module).items():
        out[name] = b.detach().clone()
    return out


def _persistent_buffers(module: nn.Module) -> dict[str, torch.Tensor]:
    """The buffers ``module.state_dict()`` holds: ``persistent=False`` ones (rotary tables and the like) are left out."""
    out = {}
    for prefix, sub in module.named_modules():
        for name, b in sub.named_buffers(recurse=False):
            if name not in sub._non_persistent_buffers_set:
                out[f"{prefix}.{name}" if prefix else name] = b
    return out


def load_full_state_dict(module: nn.Module, state_dict: Mapping[str, torch.Tensor], strict: bool = True) -> None:
    """Loads full parameters (any logical world size: each rank keeps its fragment) and buffers by name."""
    owners = _owners_by_name(module)
    missing = [k for k in owners if k not in state_dict]
    if strict and missing:
        raise KeyError(f"missing keys: {missing}")
    touched = set()
    for name, owner in owners.items():
        if name not in state_dict:
            continue
        src = state_dict[name]
        if isinstance(owner, torch.Tensor):
            with torch.no_grad():
                owner.copy_(src)
            continue
        if src.numel() != owner._orig_size.numel():
            raise ValueError(f"{name}: expected {owner._orig_size.numel()} elements, got {src.numel()}")
        n, go = owner.placement.local_numel, owner.placement.global_offset
        if n:
            flat = src.detach().to(owner.device).contiguous().view(-1)
            _native.flat_copy(owner._sharded_param_data, flat[go : go + n])
        group = owner._param_group_ref()
        if group is not None and id(group) not in touched:
            touched.add(id(group))
            group._all_gather_input_set_dtypes.clear()
            group._copy_in_shard_version = None
    buffers = _persistent_buffers(module)
    for name, b in buffers.items():
        if name in state_dict:
            with torch.no_grad():
                b.copy_(state_dict[name])
        elif strict:
            raise KeyError(f"missing buffer: {name}")
