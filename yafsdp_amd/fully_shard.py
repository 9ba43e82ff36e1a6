"""``fully_shard`` on one MI355X (mirror of ya_fsdp/fully_shard.py): the same
call contract, dynamic ``YaFSDP<Cls>`` class swap and module methods, on top of
the buffer kernels.  ``mesh`` is a logical ``(world_size, rank)`` pair (or
``None`` for a single rank) because no inter-GPU exchange is attached: with
``world_size == 1`` this is a complete sharded-data-parallel trainer for one
GPU; larger world sizes give every rank's exact layout and buffer traffic."""

from __future__ import annotations

from typing import Any, NoReturn

import torch
import torch.nn as nn

from ._api import MixedPrecisionPolicy
from ._common import resolve_device
from ._init import _get_managed_modules, _get_managed_states, _move_states_to_device, mesh_info_from
from ._param_group import YaFSDPParamGroup
from ._state import YaFSDPState, _get_module_fsdp_state

__all__ = ["UnshardHandle", "YaFSDPModule", "fully_shard"]

cls_to_fsdp_cls: dict[type, type] = {}


def fully_shard(
    module: "nn.Module | list[nn.Module]",
    *,
    mesh: Any = None,
    reshard_after_forward: bool | None = True,
    mp_policy: MixedPrecisionPolicy = MixedPrecisionPolicy(),
    ignored_params: set[nn.Parameter] | None = None,
    shard_alignment: int = 8,
    device: torch.device | str | None = None,
) -> "YaFSDPModule | list[YaFSDPModule]":
    """ya_fsdp/fully_shard.py:67-129.  A list of modules forms ONE parameter group
    whose parameters are gathered before the first of them runs forward and
    released after the last one has (ya_fsdp/_state.py:575-613)."""
    if isinstance(module, (nn.ModuleList, nn.ModuleDict)):
        raise ValueError(f"fully_shard does not support containers that do not implement forward: {module}")
    arg_module = module
    if isinstance(module, nn.Module):
        modules = (module,)
    else:
        modules = tuple(_get_root_modules(list(module)))
        if not modules or not all(isinstance(m, nn.Module) for m in modules):
            raise ValueError("fully_shard expects a module or a non-empty list of modules")
    for m in modules:
        if _get_module_fsdp_state(m) is not None:
            raise AssertionError(f"fully_shard has already been applied to {type(m).__name__}")
    mesh_info = mesh_info_from(mesh)
    device = resolve_device(device)
    auto_reshard_after_forward = reshard_after_forward is not None
    state = YaFSDPState()
    state.init(modules, device, mp_policy, auto_reshard_after_forward)
    managed_modules = _get_managed_modules(modules, _get_module_fsdp_state, ignored_params)
    params, buffers = _get_managed_states(managed_modules, ignored_params)
    _move_states_to_device(params, buffers, device)
    if params:
        names = _param_names(modules, params)
        group = YaFSDPParamGroup(params, mesh_info, device, mp_policy, shard_alignment, names=names, modules=modules)
        group.reshard_after_forward = True if reshard_after_forward is None else bool(reshard_after_forward)
        state._fsdp_param_group = group
    for m in modules:
        cls = m.__class__
        new_cls = cls_to_fsdp_cls.get(cls)
        if not new_cls:
            new_cls = type(f"YaFSDP{cls.__name__}", (YaFSDPModule, cls), {"__deepcopy__": _unimplemented_deepcopy})
            cls_to_fsdp_cls[cls] = new_cls
        m.__class__ = new_cls
    return arg_module  # type: ignore[return-value]


def _get_root_modules(modules: list) -> list:
    """The modules of the list that are not inside another module of the list
    (ya_fsdp/fully_shard.py:99-101), in list order."""
    roots = []
    for candidate in modules:
        inside = any(
            other is not candidate and any(sub is candidate for sub in other.modules())
            for other in modules
        )
        if not inside and not any(r is candidate for r in roots):
            roots.append(candidate)
    return roots


def _param_names(modules: tuple, params: list) -> list[str]:
    by_id: dict[int, str] = {}
    for k, module in enumerate(modules):
        prefix = "" if len(modules) == 1 else f"{k}."
        for n, p in module.named_parameters(remove_duplicate=False):
            by_id.setdefault(id(p), prefix + n)
    return [by_id.get(id(p), f"param{i}") for i, p in enumerate(params)]


def _unimplemented_deepcopy(*args: Any, **kwargs: Any) -> NoReturn:
    raise AssertionError("YaFSDP does not support deepcopy. Please use state dict for serialization.")


class YaFSDPModule:
    """Methods added to a module by ``fully_shard`` (ya_fsdp/fully_shard.py:138-256)."""

    def __new__(cls, *args: Any, **kwargs: Any) -> Any:
        orig_cls = cls.__mro__[2]
        self = orig_cls.__new__(orig_cls, *args, **kwargs)
        self.__init__(*args, **kwargs)
        return self

    def reshard(self) -> None:
        if group := self._get_fsdp_state()._fsdp_param_group:
            group.reshard()

    def unshard(self, async_op: bool = False) -> "UnshardHandle | None":
        state = self._get_fsdp_state()
        group = state._fsdp_param_group
        if group is not None:
            group.unshard(async_op=async_op)
        handle = _UnshardHandleImpl(group)
        if async_op:
            return handle
        handle.wait()
        return None

    def set_is_last_backward(self, is_last_backward: bool) -> None:
        self._get_fsdp_state()._state_ctx.is_last_backward = is_last_backward

    def set_requires_gradient_sync(self, requires_gradient_sync: bool, *, recurse: bool = True) -> None:
        for module in self._fsdp_modules(recurse):
            state = module._get_fsdp_state()
            if group := state._fsdp_param_group:
                group.reduce_grads = requires_gradient_sync
                if state._is_root is not None:
                    state.validate_shared_state()

    def set_reshard_after_forward(self, reshard_after_forward: bool, recurse: bool = True) -> None:
        if not isinstance(reshard_after_forward, bool):
            raise ValueError(f"reshard_after_forward should be a bool, got {type(reshard_after_forward)}")
        for module in self._fsdp_modules(recurse):
            state = module._get_fsdp_state()
            state._auto_reshard_after_forward = False
            if group := state._fsdp_param_group:
                group.reshard_after_forward = reshard_after_forward

    def set_reshard_after_backward(self, reshard_after_backward: bool, *, recurse: bool = True) -> None:
        for module in self._fsdp_modules(recurse):
            state = module._get_fsdp_state()
            if group := state._fsdp_param_group:
                group.reshard_after_backward = reshard_after_backward
                if state._is_root is not None:
                    state.validate_shared_state()

    def set_modules_to_forward_prefetch(self, modules: "list[YaFSDPModule]") -> None:
        _assert_all_fsdp_modules(modules)
        self._get_fsdp_state()._states_to_forward_prefetch = [m._get_fsdp_state() for m in modules]

    def set_modules_to_backward_prefetch(self, modules: "list[YaFSDPModule]") -> None:
        _assert_all_fsdp_modules(modules)
        self._get_fsdp_state()._states_to_backward_prefetch = [m._get_fsdp_state() for m in modules]

    def set_post_optim_event(self, event: torch.cuda.Event) -> None:
        self._get_fsdp_state()._state_ctx.post_optim_event = event

    def set_unshard_in_backward(self, unshard_in_backward: bool) -> None:
        if (group := self._get_fsdp_state()._fsdp_param_group) is not None:
            group.unshard_in_backward = unshard_in_backward

    def set_gradient_divide_factor(self, factor: float) -> None:
        if (group := self._get_fsdp_state()._fsdp_param_group) is not None:
            group.gradient_divide_factor = factor

    def set_force_sum_reduction_for_comms(self, enable: bool) -> None:
        if (group := self._get_fsdp_state()._fsdp_param_group) is not None:
            group.force_sum_reduction_for_comms = enable

    def set_reduce_copy_in_on_side_stream(self, enable: bool, *, recurse: bool = True) -> None:
        """Not part of the reference's interface.  The reference flattens a group's gradients into the reduce buffer
        on the compute stream (ya_fsdp/_param_group.py:669-708), in line with the backward GEMMs of the next group;
        with this option a backward pass that reduces runs that copy on the reduce-scatter stream instead, right in
        front of the post-reduce, and the compute stream only hands the gradients over.  Same results (the
        kernels and their order on the reduce buffer do not change); measured 4-5 % faster on a full Llama-3-8B
        pass next to GEMMs."""
        for module in self._fsdp_modules(recurse):
            if group := module._get_fsdp_state()._fsdp_param_group:
                group.reduce_copy_in_on_side_stream = bool(enable)

    def _fsdp_modules(self, recurse: bool) -> "list[YaFSDPModule]":
        mods = list(self.modules()) if recurse else [self]  # type: ignore[attr-defined]
        return [m for m in mods if isinstance(m, YaFSDPModule)]

    def _get_fsdp_state(self) -> YaFSDPState:
        if (state := _get_module_fsdp_state(self)) is None:  # type: ignore[arg-type]
            raise AssertionError(f"No YaFSDP state found on {self}")
        return state

    def _apply(self, *args: Any, **kwargs: Any) -> Any:
        """ya_fsdp/fully_shard.py:241-252."""
        self.reshard()
        ret = super()._apply(*args, **kwargs)  # type: ignore[misc]
        if not (group := self._get_fsdp_state()._fsdp_param_group):
            return ret
        with torch.no_grad():
            for fsdp_param in group.fsdp_params:
                fsdp_param.reset_sharded_param()
        return ret


class UnshardHandle:
    def wait(self) -> None:
        return


class _UnshardHandleImpl(UnshardHandle):
    def __init__(self, fsdp_param_group: YaFSDPParamGroup | None):
        self._fsdp_param_group = fsdp_param_group
        self._all_gather_result = None

    def wait(self) -> None:
        if self._fsdp_param_group is not None:
            self._all_gather_result = self._fsdp_param_group.wait_for_unshard()
            self._fsdp_param_group = None
        elif (result := self._all_gather_result) is not None:
            result.wait()


def _assert_all_fsdp_modules(modules) -> None:
    for module in modules:
        if not isinstance(module, YaFSDPModule):
            raise ValueError(f"Expects YaFSDPModule but got {type(module)}: {module}")
