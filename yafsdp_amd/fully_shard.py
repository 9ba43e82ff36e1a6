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
    """Same keyword contract and return value as ya_fsdp/fully_shard.py:67-129.  A list of modules forms ONE
    parameter group whose parameters are gathered before the first of them runs forward and released after the
    last one has (ya_fsdp/_state.py:575-613).  ``reshard_after_forward=None`` means "True, and let the root decide
    which groups may stay unsharded"."""
    roots = _group_roots(module)
    state = YaFSDPState()
    state.init(roots, resolve_device(device), mp_policy, reshard_after_forward is not None)
    managed = _get_managed_modules(roots, _get_module_fsdp_state, ignored_params)
    params, buffers = _get_managed_states(managed, ignored_params)
    _move_states_to_device(params, buffers, state._device)
    if params:
        state._fsdp_param_group = group = YaFSDPParamGroup(
            params, mesh_info_from(mesh), state._device, mp_policy, shard_alignment,
            names=_param_names(roots, params), modules=roots,
        )
        group.reshard_after_forward = reshard_after_forward is None or bool(reshard_after_forward)
    for root in roots:
        root.__class__ = _sharded_class_of(type(root))
    return module  # type: ignore[return-value]


def _group_roots(module: Any) -> tuple:
    """What one ``fully_shard`` call wraps: the module itself, or the members of a list that are not inside
    another member.  Containers without a forward and modules that are wrapped already are refused, as in
    ya_fsdp/fully_shard.py:77-80 and torch's ``contract``."""
    if isinstance(module, (nn.ModuleList, nn.ModuleDict)):
        raise ValueError(f"fully_shard does not support containers that do not implement forward: {module}")
    if isinstance(module, nn.Module):
        roots = (module,)
    else:
        members = list(module)
        if not members or not all(isinstance(m, nn.Module) for m in members):
            raise ValueError("fully_shard expects a module or a non-empty list of modules")
        roots = tuple(_get_root_modules(members))
    for root in roots:
        if _get_module_fsdp_state(root) is not None:
            raise AssertionError(f"fully_shard has already been applied to {type(root).__name__}")
    return roots


def _sharded_class_of(cls: type) -> type:
    """``YaFSDP<Cls>``: the module's own class with ``YaFSDPModule`` in front of it in the method resolution order,
    made once per class (ya_fsdp/fully_shard.py:119-127)."""
    if cls not in cls_to_fsdp_cls:
        cls_to_fsdp_cls[cls] = type(
            f"YaFSDP{cls.__name__}", (YaFSDPModule, cls), {"__deepcopy__": _unimplemented_deepcopy}
        )
    return cls_to_fsdp_cls[cls]


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
    """The methods a module gains from ``fully_shard`` (names, arguments and effects of
    ya_fsdp/fully_shard.py:138-256).  Every setter is a write to the module's parameter group or to the state the
    groups of one model share; those that change what a shared buffer must hold re-run the buffer validation once
    the root has assigned buffers."""

    def __new__(cls, *args: Any, **kwargs: Any) -> Any:
        # YaFSDP<Cls> -> YaFSDPModule -> Cls: constructing the swapped class constructs a plain Cls
        plain = cls.__mro__[2]
        obj = plain.__new__(plain, *args, **kwargs)
        obj.__init__(*args, **kwargs)
        return obj

    # ---- lookups the methods share -------------------------------------------------------------
    def _get_fsdp_state(self) -> YaFSDPState:
        state = _get_module_fsdp_state(self)  # type: ignore[arg-type]
        if state is None:
            raise AssertionError(f"No YaFSDP state found on {self}")
        return state

    def _fsdp_modules(self, recurse: bool) -> "list[YaFSDPModule]":
        """This module, or every wrapped module at or below it, in ``nn.Module.modules()`` order."""
        candidates = self.modules() if recurse else (self,)  # type: ignore[attr-defined]
        return [m for m in candidates if isinstance(m, YaFSDPModule)]

    def _own_group(self) -> "YaFSDPParamGroup | None":
        return self._get_fsdp_state()._fsdp_param_group

    def _write_to_groups(self, recurse: bool, attr: str, value: Any, *, revalidate: bool = False) -> None:
        for module in self._fsdp_modules(recurse):
            state = module._get_fsdp_state()
            if (group := state._fsdp_param_group) is None:
                continue
            setattr(group, attr, value)
            if revalidate and state._is_root is not None:  # buffers are assigned: check they still suffice
                state.validate_shared_state()

    # ---- gathering and releasing by hand -------------------------------------------------------
    def reshard(self) -> None:
        if (group := self._own_group()) is not None:
            group.reshard()

    def unshard(self, async_op: bool = False) -> "UnshardHandle | None":
        group = self._own_group()
        if group is not None:
            group.unshard(async_op=async_op)
        handle = _UnshardHandleImpl(group)
        if async_op:
            return handle
        handle.wait()
        return None

    # ---- per-group switches --------------------------------------------------------------------
    def set_requires_gradient_sync(self, requires_gradient_sync: bool, *, recurse: bool = True) -> None:
        self._write_to_groups(recurse, "reduce_grads", requires_gradient_sync, revalidate=True)

    def set_reshard_after_backward(self, reshard_after_backward: bool, *, recurse: bool = True) -> None:
        self._write_to_groups(recurse, "reshard_after_backward", reshard_after_backward, revalidate=True)

    def set_reshard_after_forward(self, reshard_after_forward: bool, recurse: bool = True) -> None:
        if not isinstance(reshard_after_forward, bool):
            raise ValueError(f"reshard_after_forward should be a bool, got {type(reshard_after_forward)}")
        for module in self._fsdp_modules(recurse):
            module._get_fsdp_state()._auto_reshard_after_forward = False  # an explicit choice: the root keeps it
        self._write_to_groups(recurse, "reshard_after_forward", reshard_after_forward)

    def set_unshard_in_backward(self, unshard_in_backward: bool) -> None:
        self._write_to_groups(False, "unshard_in_backward", unshard_in_backward)

    def set_gradient_divide_factor(self, factor: float) -> None:
        self._write_to_groups(False, "gradient_divide_factor", factor)

    def set_force_sum_reduction_for_comms(self, enable: bool) -> None:
        self._write_to_groups(False, "force_sum_reduction_for_comms", enable)

    def set_reduce_copy_in_on_side_stream(self, enable: bool, *, recurse: bool = True) -> None:
        """Not part of the reference's interface.  The reference flattens a group's gradients into the reduce buffer
        on the compute stream (ya_fsdp/_param_group.py:669-708), in line with the backward GEMMs of the next group;
        with this option a backward pass that reduces runs that copy on the reduce-scatter stream instead, right in
        front of the post-reduce, and the compute stream only hands the gradients over.  Same results (the
        kernels and their order on the reduce buffer do not change); measured 4-5 % faster on a full Llama-3-8B
        pass next to GEMMs."""
        self._write_to_groups(recurse, "reduce_copy_in_on_side_stream", bool(enable))

    # ---- state shared by the groups of one model -----------------------------------------------
    def set_is_last_backward(self, is_last_backward: bool) -> None:
        self._get_fsdp_state()._state_ctx.is_last_backward = is_last_backward

    def set_post_optim_event(self, event: torch.cuda.Event) -> None:
        self._get_fsdp_state()._state_ctx.post_optim_event = event

    def set_modules_to_forward_prefetch(self, modules: "list[YaFSDPModule]") -> None:
        self._get_fsdp_state()._states_to_forward_prefetch = _states_of(modules)

    def set_modules_to_backward_prefetch(self, modules: "list[YaFSDPModule]") -> None:
        self._get_fsdp_state()._states_to_backward_prefetch = _states_of(modules)

    def _apply(self, *args: Any, **kwargs: Any) -> Any:
        """``.to()`` / ``.float()`` / ``.cuda()`` act on the registered (sharded) parameters, after which each
        parameter's shard bookkeeping is rebuilt from what ``nn.Module._apply`` left (ya_fsdp/fully_shard.py:241-252)."""
        self.reshard()
        ret = super()._apply(*args, **kwargs)  # type: ignore[misc]
        if (group := self._own_group()) is not None:
            with torch.no_grad():
                for fsdp_param in group.fsdp_params:
                    fsdp_param.reset_sharded_param()
        return ret


class UnshardHandle:
    """What ``unshard(async_op=True)`` returns: ``wait()`` makes the current stream wait for the gathered
    parameters."""

    def wait(self) -> None:
        return


class _UnshardHandleImpl(UnshardHandle):
    def __init__(self, fsdp_param_group: YaFSDPParamGroup | None):
        self._fsdp_param_group = fsdp_param_group  # dropped at the first wait: a handle must not keep a group alive
        self._all_gather_result = None

    def wait(self) -> None:
        group, self._fsdp_param_group = self._fsdp_param_group, None
        if group is not None:
            self._all_gather_result = group.wait_for_unshard()
        elif self._all_gather_result is not None:
            self._all_gather_result.wait()


def _assert_all_fsdp_modules(modules) -> None:
    for module in modules:
        if not isinstance(module, YaFSDPModule):
            raise ValueError(f"Expects YaFSDPModule but got {type(module)}: {module}")


def _states_of(modules) -> "list[YaFSDPState]":
    _assert_all_fsdp_modules(modules)
    return [module._get_fsdp_state() for module in modules]
