"""Module discovery for ``fully_shard`` (mirror of ya_fsdp/_init.py:100-220):
which submodules a call manages, in which order their parameters enter the flat
buffer (post-order DFS over submodules, then ``named_parameters(recurse=False)``),
and moving them to the device."""

from __future__ import annotations

import itertools

import torch
import torch.nn as nn

from ._common import FSDPMeshInfo


def mesh_info_from(mesh) -> FSDPMeshInfo:
    """The reference takes a 1-D ``DeviceMesh`` (ya_fsdp/fully_shard.py:81-85).
    On one GPU the mesh is a logical ``(world_size, rank)`` pair; ``None`` is the
    single-rank default."""
    if mesh is None:
        return FSDPMeshInfo(1, 0)
    if isinstance(mesh, FSDPMeshInfo):
        return mesh
    if isinstance(mesh, (tuple, list)) and len(mesh) == 2:
        return FSDPMeshInfo(int(mesh[0]), int(mesh[1]))
    ndim = getattr(mesh, "ndim", None)
    if ndim is not None:
        if ndim != 1:
            raise ValueError(f"fully_shard expects a 1D DeviceMesh but got {mesh}")
        return FSDPMeshInfo(int(mesh.size(0)), int(mesh.get_local_rank(0)))
    raise ValueError(f"mesh must be None, (world_size, rank), FSDPMeshInfo or a 1-D DeviceMesh, got {mesh!r}")


def _get_managed_modules(root_modules: tuple, get_state, ignored_params: set | None = None) -> list[nn.Module]:
    """ya_fsdp/_init.py:123-153 (post-order DFS; nested ``fully_shard`` modules
    are left to their own state)."""
    modules: list[nn.Module] = []
    root_modules_set = set(root_modules)
    visited: set[nn.Module] = set()

    def dfs(module: nn.Module) -> None:
        if module not in root_modules_set and get_state(module) is not None:
            return
        visited.add(module)
        for submodule in module.children():
            if submodule not in visited:
                dfs(submodule)
        modules.append(module)

    for root in root_modules:
        dfs(root)
    if ignored_params is None:
        return modules
    return _adjust_managed_modules(modules, ignored_params)


def _ignore_module(module: nn.Module, ignored_params: set, decision: dict) -> bool:
    """A module drops out of the managed set only if it owns no buffer, every parameter it owns is ignored and
    every child drops out too (the rule of ya_fsdp/_init.py:79-108); ``decision`` memoises per module."""
    if module not in decision:
        decision[module] = (
            next(iter(module.buffers(recurse=False)), None) is None
            and all(param in ignored_params for param in module.parameters(recurse=False))
            and all(_ignore_module(child, ignored_params, decision) for child in module.children())
        )
    return decision[module]


def _adjust_managed_modules(modules: list[nn.Module], ignored_params: set) -> list[nn.Module]:
    decision: dict[nn.Module, bool] = {}
    return [m for m in modules if not _ignore_module(m, ignored_params, decision)]


def _get_managed_states(modules: list[nn.Module], ignored_params: set | None = None):
    """The parameters and buffers that the given modules own directly, each object once, in module order
    (what ya_fsdp/_init.py:164-189 collects).  A 0-d parameter cannot be split along dim 0 and is refused."""
    skip = ignored_params or set()
    params: dict[nn.Parameter, None] = {}  # insertion-ordered, keyed by identity (a tensor hashes by id)
    buffers: dict[torch.Tensor, None] = {}
    for module in modules:
        for name, param in module.named_parameters(recurse=False):
            if param in skip or param in params:
                continue
            if param.dim() == 0:
                raise ValueError(
                    f"fully_shard doesn't support scalar parameters. Change {name} to a 1D tensor with numel equal to 1."
                )
            params[param] = None
        buffers.update(dict.fromkeys(module.buffers(recurse=False)))
    return list(params), list(buffers)


def _move_states_to_device(params, buffers, device: torch.device) -> None:
    """ya_fsdp/_init.py:192-220 for plain tensors."""
    for tensor in itertools.chain(params, buffers):
        if tensor.device == device:
            continue
        if tensor.is_meta:
            # deferred initialisation (:205-211): an uninitialised tensor of the same shape takes the meta tensor's
            # place; the caller fills the sharded parameters in afterwards
            with torch.no_grad():  # avoid autograd increasing C++ refcount by 1
                empty = torch.empty_like(tensor, device=device)
                if isinstance(tensor, nn.Parameter):
                    empty = nn.Parameter(empty, requires_grad=tensor.requires_grad)
            torch.utils.swap_tensors(tensor, empty)
        else:
            tensor.data = tensor.to(device)
