"""Per-parameter bookkeeping of a parameter group: every tensor here is a VIEW
into one of the group's flat buffers (mirror of ya_fsdp/_param.py, restricted to
what the buffer path touches: no DTensor wrapping, no module attribute swaps).
"""

from __future__ import annotations

import weakref
from dataclasses import dataclass, field

import torch
import torch.nn as nn

from ._api import MixedPrecisionPolicy
from ._common import FSDPMeshInfo, ShardedState
from ._layout import RaggedShard


@dataclass
class ParamModuleInfo:
    """Where a parameter is registered, so that the sharded / unsharded views
    can be swapped in with ``setattr`` (ya_fsdp/_param.py:20-31); shared
    (tied) registrations are listed as well."""

    module: nn.Module
    param_name: str
    shared_modules: list[nn.Module] = field(default_factory=list)
    shared_param_names: list[str] = field(default_factory=list)


class YaFSDPParam:
    orig_dtype: torch.dtype
    param_dtype: torch.dtype | None
    reduce_dtype: torch.dtype | None

    def __init__(
        self, param: torch.Tensor, mesh_info: FSDPMeshInfo, device: torch.device, name: str | None = None,
        module_info: ParamModuleInfo | None = None,
    ):
        if param.device != device:
            raise AssertionError(
                f"Expects the parameter to already be moved to device {device} but got {param.device}"
            )  # ya_fsdp/_param.py:69-72
        if not param.is_contiguous():
            raise NotImplementedError(
                f"YaFSDP does not support non-contiguous parameters yet: {param.shape=} {param.stride()=}"
            )  # ya_fsdp/_param.py:74-77
        if param.dim() == 0:
            raise ValueError("Change the scalar parameter to a 1D tensor with numel equal to 1.")  # _init.py:156-161
        self.param = param
        self.param_data = param
        self._module_info = module_info
        self.mesh_info = mesh_info
        self.device = device
        self._param_fqn = name
        self._orig_size = param.size()
        self.requires_grad = bool(param.requires_grad)
        self.unsharded_accumulated_grad: torch.Tensor | None = None
        self._unsharded_accumulated_grad: torch.Tensor | None = None
        self.sharded_state = ShardedState.SHARDED

    # ---- dtype clamping (ya_fsdp/_param.py:170-183) ----------------------------
    def init_dtype_attrs(self, mp_policy: MixedPrecisionPolicy) -> None:
        param_dtype, reduce_dtype = mp_policy.param_dtype, mp_policy.reduce_dtype
        self.orig_dtype = self.param.dtype
        if reduce_dtype == param_dtype:
            reduce_dtype = None
        if param_dtype == self.orig_dtype:
            param_dtype = None
        self.param_dtype = param_dtype
        self.reduce_dtype = reduce_dtype

    # ---- views (ya_fsdp/_param.py:84-168, 197-231) ------------------------------
    @torch.no_grad()
    def init_sharded_param(
        self,
        sharded_param_data: torch.Tensor,
        sharded_param_grad: torch.Tensor | None,
        global_offset: int,
        shard_numels: tuple[int, ...],
    ) -> None:
        self.placement = RaggedShard(
            local_numel=sharded_param_data.numel(), global_offset=global_offset, shard_numels=shard_numels
        )
        self.sharded_numel = sharded_param_data.numel()
        self._sharded_param_data = sharded_param_data
        self.sharded_param = nn.Parameter(sharded_param_data, requires_grad=self.requires_grad)
        self.sharded_param._yafsdp_param = weakref.ref(self)  # lets flat-shard optimizers find the owner
        self.sharded_param_grad = sharded_param_grad if self.requires_grad else None
        del self.param, self.param_data  # the group's flat shard now owns the values
        self._setattr_on_modules(self.sharded_param)

    def init_all_gather_input(self, all_gather_input: torch.Tensor) -> None:
        self._all_gather_input = all_gather_input

    def init_reduce_scatter_output(self, reduce_scatter_output: torch.Tensor) -> None:
        self.reduce_scatter_output = reduce_scatter_output

    def init_unsharded_param(
        self, all_gather_output: torch.Tensor, reduce_scatter_input: torch.Tensor | None
    ) -> None:
        unsharded_tensor = all_gather_output.view(self._orig_size)  # zero-copy copy-out
        self.unsharded_param = nn.Parameter(unsharded_tensor, requires_grad=self.requires_grad)
        self.unsharded_param._yafsdp_param = weakref.ref(self)
        if self.requires_grad:
            assert reduce_scatter_input is not None
            self._unsharded_accumulated_grad = reduce_scatter_input.view(self._orig_size)
        else:
            self._unsharded_accumulated_grad = None

    def set_all_gather_input(self) -> None:
        """Hook of ya_fsdp/_param.py:281-291 for tensor subclasses with
        ``fsdp_pre_all_gather``; plain tensors have nothing to do."""
        if self.sharded_state != ShardedState.SHARDED:
            raise AssertionError(f"Expects to be in SHARDED, not {self.sharded_state}")

    def to_sharded(self) -> None:
        self._setattr_on_modules(self.sharded_param)
        self.sharded_state = ShardedState.SHARDED

    def to_unsharded(self) -> None:
        self._setattr_on_modules(self.unsharded_param)
        self.sharded_state = ShardedState.UNSHARDED

    def _setattr_on_modules(self, param: nn.Parameter) -> None:
        """ya_fsdp/_param.py:259-268."""
        info = self._module_info
        if info is None:
            return
        unsafe_setattr_param(info.module, info.param_name, param)
        for shared_module, shared_param_name in zip(info.shared_modules, info.shared_param_names):
            unsafe_setattr_param(shared_module, shared_param_name, param)

    def reset_sharded_param(self) -> None:
        """Re-sync after ``module._apply`` replaced the registered parameter
        (ya_fsdp/_param.py:345-357): copy its values back into the flat shard."""
        info = self._module_info
        if info is None:
            return
        new_param = getattr(info.module, info.param_name)
        if new_param.data_ptr() != self._sharded_param_data.data_ptr() and self.sharded_numel > 0:
            from . import _native

            if new_param.device != self._sharded_param_data.device or new_param.numel() != self.sharded_numel:
                raise NotImplementedError(
                    "moving a sharded module to another device or changing its parameter sizes is not supported"
                )
            _native.flat_copy(self._sharded_param_data, new_param.detach().contiguous().view(-1))
        self.sharded_param = nn.Parameter(self._sharded_param_data, requires_grad=self.sharded_param.requires_grad)
        self.sharded_param._yafsdp_param = weakref.ref(self)
        self._setattr_on_modules(self.sharded_param)

    @property
    def unsharded_grad_data(self) -> torch.Tensor:
        grad = self.unsharded_param.grad
        if grad is None:
            raise AssertionError("Expects unsharded_param.grad to not be None")
        return grad

    def __repr__(self) -> str:
        return f"YaFSDPParam(fqn={self._param_fqn}, orig_size={self._orig_size})"


def unsafe_setattr_param(module: nn.Module, param_name: str, param: nn.Parameter) -> None:
    """ya_fsdp/_param.py:363-372: skip ``nn.Module.__setattr__`` checks when the
    module does not override it."""
    if getattr(module.__setattr__, "__func__", None) is nn.Module.__setattr__:
        module._parameters[param_name] = param
    else:
        setattr(module, param_name, param)
