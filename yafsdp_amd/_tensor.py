"""``RaggedShardDTensor``: what a sharded parameter (and its gradient) is after
``fully_shard`` (mirror of ya_fsdp/_tensor.py:54-432).

The tensor *stands for* the whole parameter - ``size()`` is the parameter's
original shape - while it *holds* this rank's 1-D fragment of it: a view into
the group's flat master (or gradient) shard, ``[global_offset, global_offset +
local_numel)`` of the parameter flattened.  ``to_local()``, ``placements``,
``full_tensor()`` and the three ``torch.distributed.checkpoint`` hooks are those
of the reference; tensor ops reach it through the same allow-list
(``__torch_dispatch__``), which forwards optimizer, clipping and initialisation
ops to the local fragments, so ``torch.optim`` (foreach and fused),
``torch.nn.utils.clip_grad_norm_`` and ``Module.state_dict()`` work on the
sharded parameters as they do with the reference.

What differs on one GPU (no process group, the shard world is logical):

* the spec's ``mesh`` is the logical ``FSDPMeshInfo`` (size, rank), not a ``DeviceMesh``;
* ``_foreach_norm`` returns the norms of the local fragments as plain tensors (the reference wraps them in a
  ``DTensor`` with a ``_NormPartial`` placement, which the next op reduces over the mesh): with a logical world
  size of 1 that is the full norm, otherwise this rank's part of it;
* ``normal_`` / ``uniform_`` / ``rand_like`` draw from the device generator for the local fragment (the reference
  offsets the generator per rank through DTensor's RNG tracker);
* ``full_tensor()`` with a logical world size above 1 reads the other logical ranks' fragments, which live in the
  same process: they have to be introduced first (``connect_logical_ranks``);
* ``copy_`` also accepts a plain tensor of the parameter's full shape and takes this rank's fragment of it.
"""

from __future__ import annotations

import operator
import warnings
import weakref
from dataclasses import dataclass, field
from functools import reduce
from typing import Any, Sequence

import torch
from torch.distributed.tensor._dtensor_spec import TensorMeta
from torch.optim.optimizer import _foreach_supported_types as _optim_foreach_supported_types
from torch.utils._foreach_utils import _foreach_supported_types as _util_foreach_supported_types

from ._common import FSDPMeshInfo
from ._layout import RaggedShard

__all__ = ["RaggedShardDTensor", "RaggedShardSpec", "connect_logical_ranks", "local_tensor"]


@dataclass(frozen=True)
class RaggedShardSpec:
    """Stands where ``DTensorSpec`` stands in the reference: mesh, placements and the metadata of the whole
    parameter.  ``owner`` (not part of equality) leads back to the ``YaFSDPParam`` for ``full_tensor()``."""

    mesh: FSDPMeshInfo
    placements: tuple[RaggedShard, ...]
    tensor_meta: TensorMeta
    # set only on a group's own parameter / gradient fragments: weakref to the YaFSDPParam and which of its two
    # fragments this is ("param" or "grad"); tensors derived by ops (clones, optimizer state) carry neither
    owner: Any = field(default=None, compare=False, repr=False)
    kind: str = field(default="", compare=False, repr=False)

    def __reduce__(self) -> Any:  # pickles without the back-reference
        return (RaggedShardSpec, (self.mesh, self.placements, self.tensor_meta))

    def derived(self, dtype: torch.dtype | None = None) -> "RaggedShardSpec":
        meta = self.tensor_meta
        if dtype is not None and dtype != meta.dtype:
            meta = TensorMeta(meta.shape, meta.stride, dtype)
        return RaggedShardSpec(self.mesh, self.placements, meta)


def local_tensor(t: torch.Tensor) -> torch.Tensor:
    """The local fragment of a ``RaggedShardDTensor``; any other tensor as it is."""
    return t._local_tensor if isinstance(t, RaggedShardDTensor) else t


def plain_tensor(t: torch.Tensor) -> torch.Tensor:
    """The plain tensor at the bottom of a local fragment: a tensor-subclass parameter is sharded as an instance of
    its subclass whose first inner tensor is the fragment of the flat shard (ya_fsdp/_param.py:145-152)."""
    while type(t) not in (torch.Tensor, torch.nn.Parameter) and hasattr(t, "__tensor_flatten__"):
        t = getattr(t, t.__tensor_flatten__()[0][0])
    return t


def _locals(ts: Sequence[torch.Tensor]) -> list[torch.Tensor]:
    return [local_tensor(t) for t in ts]


def _written(ts: Sequence[torch.Tensor]) -> None:
    """In-place ops that run inside ``__torch_dispatch__`` do not bump version counters (the dispatch keys that do
    are already behind us).  The local fragments are views of a group's flat shard, and the buffer path compares
    that shard's version to know whether its 16-bit copy or its fused gradient norm is stale: bump by hand."""
    ts = [t for t in ts if isinstance(t, torch.Tensor)]
    if ts:
        torch.autograd.graph.increment_version(ts)


class RaggedShardDTensor(torch.Tensor):
    _local_tensor: torch.Tensor
    _spec: RaggedShardSpec
    __slots__ = ["_local_tensor", "_spec"]

    @staticmethod
    def __new__(cls, local_tensor: torch.Tensor, spec: RaggedShardSpec, *, requires_grad: bool) -> "RaggedShardDTensor":
        if local_tensor.requires_grad and not requires_grad:
            warnings.warn(
                "To construct a RaggedShardDTensor from torch.Tensor, it's recommended to "
                "use local_tensor.detach() and make requires_grad consistent.",
                stacklevel=1,
            )
        assert spec.tensor_meta is not None, "TensorMeta should not be None!"
        r = torch.Tensor._make_wrapper_subclass(
            cls,
            spec.tensor_meta.shape,
            strides=spec.tensor_meta.stride,
            dtype=local_tensor.dtype,
            device=local_tensor.device,
            layout=local_tensor.layout,
            requires_grad=requires_grad,
        )
        r._spec = spec
        r._local_tensor = local_tensor
        return r

    def __repr__(self) -> str:  # type: ignore[override]
        return (f"RaggedShardDTensor(local_tensor={self._local_tensor}, device_mesh={self._spec.mesh}, "
                f"placements={self._spec.placements})")

    def __tensor_flatten__(self) -> Any:
        return ["_local_tensor"], (self._spec, self.requires_grad)

    @staticmethod
    def __tensor_unflatten__(inner_tensors: Any, flatten_spec: Any, outer_size: Any, outer_stride: Any) -> Any:
        assert flatten_spec is not None, "Expecting spec to be not None from `__tensor_flatten__` return value!"
        spec, requires_grad = flatten_spec
        meta = TensorMeta(shape=outer_size, stride=outer_stride, dtype=spec.tensor_meta.dtype)
        return RaggedShardDTensor(
            inner_tensors["_local_tensor"], RaggedShardSpec(spec.mesh, spec.placements, meta, spec.owner, spec.kind),
            requires_grad=requires_grad,
        )

    # ---- ops: the reference's allow-list (ya_fsdp/_tensor.py:122-316) ----------------------------------------
    @classmethod
    def __torch_dispatch__(cls, func: Any, types: Any, args: Any = (), kwargs: Any = None) -> Any:  # noqa: PLR0911, PLR0912
        kwargs = {} if kwargs is None else kwargs
        aten = torch.ops.aten
        if func == aten.detach.default:
            (arg,) = args
            return RaggedShardDTensor(arg._local_tensor, arg._spec, requires_grad=False)
        if func == aten.copy_.default:
            dst, src, *rest = args
            if not isinstance(src, RaggedShardDTensor) and isinstance(src, torch.Tensor):
                full_shape = tuple(dst._spec.tensor_meta.shape)
                if tuple(src.shape) == full_shape and tuple(src.shape) != tuple(dst._local_tensor.shape):
                    # a plain tensor of the whole parameter: this rank keeps its fragment of it
                    p = dst._spec.placements[0]
                    src = src.reshape(-1)[p.global_offset : p.global_offset + p.local_numel] if p.local_numel else src.reshape(-1)[:0]
            func(dst._local_tensor, local_tensor(src), *rest, **kwargs)
            _written([dst._local_tensor])
            return dst
        if func in (aten.log_.default, aten.zero_.default, aten.mul_.Tensor, aten.fill_.Scalar):
            arg, *rest = args
            func(arg._local_tensor, *_locals_any(rest), **kwargs)
            _written([arg._local_tensor])
            return arg
        if func in (
            aten.clone.default, aten._to_copy.default, aten.empty_like.default, aten.zeros_like.default,
            aten.new_zeros.default, aten.new_empty.default, aten.exp.default, aten.expm1.default, aten.log.default,
            aten.neg.default, aten.clamp.default, aten.mul.Tensor, aten.add.Tensor,
        ):
            arg, *rest = args
            if func in (aten.new_zeros.default, aten.new_empty.default):
                # the size argument names the whole parameter; the result is another fragment-sized tensor
                rest = [list(arg._local_tensor.shape), *rest[1:]]
            out = func(arg._local_tensor, *_locals_any(rest), **kwargs)
            return RaggedShardDTensor(out, arg._spec.derived(out.dtype), requires_grad=arg.requires_grad)
        if func in (aten.normal_.default, aten.uniform_.default):
            arg, *rest = args
            func(arg._local_tensor, *rest, **kwargs)
            _written([arg._local_tensor])
            return arg
        if func == aten.rand_like.default:
            arg, *rest = args
            out = func(arg._local_tensor, *rest, **kwargs)
            return RaggedShardDTensor(out, arg._spec.derived(out.dtype), requires_grad=arg.requires_grad)
        if func == aten._foreach_sqrt.default:
            (ts,) = args
            outs = func(_locals(ts), **kwargs)
            assert all(not t.requires_grad for t in ts)
            return [RaggedShardDTensor(o, t._spec.derived(), requires_grad=False) for t, o in zip(ts, outs)]
        if func == aten._foreach_norm.Scalar:
            ts, norm_type, *rest = args
            assert all(not t.requires_grad for t in ts)
            return func(_locals(ts), norm_type, *rest, **kwargs)  # norms of the local fragments (see the module text)
        if func == aten._foreach_zero_.default:
            (ts,) = args
            func(_locals(ts), **kwargs)
            _written(_locals(ts))
            return None
        if func in (aten._foreach_add_.Scalar, aten._foreach_mul_.Scalar, aten._foreach_div_.Scalar,
                    aten._foreach_div_.ScalarList, aten._foreach_mul_.ScalarList, aten._foreach_add_.ScalarList):
            ts, scale = args
            func(_locals(ts), scale, **kwargs)
            _written(_locals(ts))
            return None
        if func in (aten._foreach_mul_.Tensor, aten._foreach_div_.Tensor):
            ts, tensor = args
            func(_locals(ts), local_tensor(tensor), **kwargs)
            _written(_locals(ts))
            return None
        if func in (aten._foreach_add_.List, aten._foreach_mul_.List, aten._foreach_div_.List):
            a, b = args
            func(_locals(a), _locals(b), **kwargs)
            _written(_locals(a))
            return None
        if func == aten._foreach_lerp_.Scalar:
            a, b, scalar = args
            func(_locals(a), _locals(b), scalar, **kwargs)
            _written(_locals(a))
            return None
        if func in (aten._foreach_addcmul_.Scalar, aten._foreach_addcdiv_.Scalar, aten._foreach_addcdiv_.ScalarList,
                    aten._foreach_addcmul_.ScalarList, aten._foreach_addcdiv_.Tensor, aten._foreach_addcmul_.Tensor):
            a, b, c, scalar = args
            func(_locals(a), _locals(b), _locals(c), scalar, **kwargs)
            _written(_locals(a))
            return None
        if func in (aten._fused_adam_.default, aten._fused_adamw_.default):
            a1, a2, a3, a4, a5, a6 = args
            assert len(a5) == 0
            func(_locals(a1), _locals(a2), _locals(a3), _locals(a4), a5, a6, **kwargs)
            _written(_locals(a1) + _locals(a3) + _locals(a4))
            return None
        raise NotImplementedError(f"RaggedShardDTensor dispatch for {func} is not implemented yet.")

    # ---- the DTensor-like surface (ya_fsdp/_tensor.py:318-363) ------------------------------------------------
    def to_local(self) -> torch.Tensor:
        if torch.is_grad_enabled():
            raise NotImplementedError
        return self._local_tensor

    @property
    def device_mesh(self) -> FSDPMeshInfo:
        return self._spec.mesh

    @property
    def placements(self) -> tuple[RaggedShard, ...]:
        return self._spec.placements

    def full_tensor(self) -> torch.Tensor:
        """The whole parameter, assembled from the ranks' fragments in rank order into a new tensor (the
        reference all-gathers into ``full.split(shard_numels)``, ya_fsdp/_tensor.py:341-363)."""
        from . import _native

        placement = self._spec.placements[0]
        shard_numels = placement.shard_numels
        own = plain_tensor(self._local_tensor)
        full = own.new_empty(sum(shard_numels))
        rank = self._spec.mesh.shard_mesh_rank
        pieces = full.split(list(shard_numels))
        if len(shard_numels) == 1:
            locals_by_rank = [own]
        else:
            owner = self._spec.owner() if self._spec.owner is not None else None
            peers = getattr(owner, "_logical_peers", None)
            if peers is None:
                raise RuntimeError(
                    f"full_tensor() of a tensor sharded over {len(shard_numels)} logical ranks needs the other ranks' "
                    "fragments. On one GPU they live in this process: it works for the parameters and gradients of "
                    "fully_shard modules once the ranks' modules have been introduced to each other with "
                    "yafsdp_amd.connect_logical_ranks([module_rank0, module_rank1, ...])."
                )
            locals_by_rank = []
            for k, ref in enumerate(peers):
                peer = ref()
                if peer is None:
                    raise RuntimeError(f"logical rank {k} of this parameter no longer exists")
                if k == rank:
                    locals_by_rank.append(own)
                elif self._spec.kind == "grad":
                    locals_by_rank.append(plain_tensor(peer.sharded_param_grad._local_tensor))
                else:
                    locals_by_rank.append(peer._sharded_param_data)
        for piece, src in zip(pieces, locals_by_rank):
            if piece.numel() != src.numel():
                raise RuntimeError(f"fragment of {src.numel()} elements where the layout says {piece.numel()}")
            if piece.numel():
                _native.flat_copy(piece, src.detach())
        return full.view(self.size())

    # ---- torch.distributed.checkpoint hooks (ya_fsdp/_tensor.py:365-432) --------------------------------------
    def _chunk(self) -> tuple[torch.Size, torch.Size]:
        placement = self._spec.placements[0]
        if placement.local_numel == 0:
            offsets = torch.Size((self.numel(),))  # an empty fragment sits at the end of the flattened parameter
        else:
            offsets = torch.Size((placement.global_offset,))
        return offsets, torch.Size((placement.local_numel,))

    def __create_write_items__(self, fqn: str, object: Any) -> list:  # noqa: A002  (the protocol's argument name)
        from torch.distributed.checkpoint.metadata import ChunkStorageMetadata, MetadataIndex, TensorProperties
        from torch.distributed.checkpoint.planner import TensorWriteData, WriteItem, WriteItemType

        assert object is self
        offsets, sizes = self._chunk()
        return [
            WriteItem(
                index=MetadataIndex(fqn, offsets),
                type=WriteItemType.SHARD,
                tensor_data=TensorWriteData(
                    chunk=ChunkStorageMetadata(offsets=offsets, sizes=sizes),
                    properties=TensorProperties.create_from_tensor(plain_tensor(self._local_tensor)),
                    size=torch.Size((reduce(operator.mul, self.size(), 1),)),
                ),
            )
        ]

    def __create_chunk_list__(self) -> list:
        from torch.distributed.checkpoint.metadata import ChunkStorageMetadata

        offsets, sizes = self._chunk()
        return [ChunkStorageMetadata(offsets=offsets, sizes=sizes)]

    def __get_tensor_shard__(self, index: int) -> torch.Tensor:
        # the plain fragment of the flat shard: what a tensor-subclass parameter wraps is written as its values
        return plain_tensor(self._local_tensor)


def _locals_any(args: Sequence[Any]) -> list[Any]:
    return [local_tensor(a) if isinstance(a, torch.Tensor) else a for a in args]


def connect_logical_ranks(modules: Sequence[torch.nn.Module]) -> None:
    """Introduce the logical ranks of one model to each other: ``modules[k]`` is the copy of the model wrapped with
    ``mesh=(W, k)``.  Afterwards ``full_tensor()`` of any sharded parameter (or gradient) can read the other ranks'
    fragments.  One GPU only: in the reference this is an all-gather over the shard process group."""
    from .optim import fsdp_param_groups

    per_rank = [fsdp_param_groups(m) for m in modules]
    if len({len(gs) for gs in per_rank}) != 1:
        raise ValueError("the modules do not hold the same number of parameter groups")
    for groups in zip(*per_rank):
        w = groups[0].mesh_info.shard_mesh_size
        if len(groups) != w or [g.mesh_info.shard_mesh_rank for g in groups] != list(range(w)):
            raise ValueError(f"expected the {w} logical ranks of a group in rank order, got "
                             f"{[(g.mesh_info.shard_mesh_size, g.mesh_info.shard_mesh_rank) for g in groups]}")
        if len({len(g.fsdp_params) for g in groups}) != 1:
            raise ValueError("the ranks' groups differ in their parameters")
        for fsdp_params in zip(*(g.fsdp_params for g in groups)):
            refs = [weakref.ref(p) for p in fsdp_params]
            for p in fsdp_params:
                p._logical_peers = refs


torch.serialization.add_safe_globals([RaggedShardDTensor, RaggedShardSpec, RaggedShard, FSDPMeshInfo, TensorMeta])

# torch.optim and clip_grad_norm_ pick their foreach implementations only for tensor types on these lists
# (ya_fsdp/_tensor.py:437-444)
if RaggedShardDTensor not in _optim_foreach_supported_types:
    _optim_foreach_supported_types.append(RaggedShardDTensor)
if RaggedShardDTensor not in _util_foreach_supported_types:
    _util_foreach_supported_types.append(RaggedShardDTensor)
