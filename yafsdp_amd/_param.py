"""Per-parameter bookkeeping of a parameter group: every tensor here is a VIEW
into one of the group's flat buffers (mirror of ya_fsdp/_param.py, restricted to
what the buffer path touches).  The sharded parameter and its gradient are
``RaggedShardDTensor`` wrappers around 1-D views of the flat master / gradient
shard (ya_fsdp/_param.py:142-151).
"""

from __future__ import annotations

import weakref
from dataclasses import dataclass, field

import torch
import torch.nn as nn

from ._api import MixedPrecisionPolicy
from ._common import FSDPMeshInfo, ShardedState
from ._layout import RaggedShard
from ._tensor import RaggedShardDTensor, RaggedShardSpec, TensorMeta, local_tensor


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
        self._sharding_spec = RaggedShardSpec(  # :136-140 with the logical mesh in the DeviceMesh's place
            self.mesh_info, (self.placement,), TensorMeta(self._orig_size, self.param.stride(), self.param.dtype),
            weakref.ref(self), "param",
        )
        self.sharded_param = nn.Parameter(self.to_sharded_dtensor(sharded_param_data), requires_grad=self.requires_grad)
        self.sharded_param._yafsdp_param = weakref.ref(self)  # lets flat-shard optimizers find the owner
        if self.requires_grad:
            assert sharded_param_grad is not None
            self.sharded_param_grad = self.to_sharded_dtensor(sharded_param_grad, "grad")
        else:
            self.sharded_param_grad = None
        del self.param, self.param_data  # the group's flat shard now owns the values
        self._setattr_on_modules(self.sharded_param)

    def to_sharded_dtensor(self, tensor: torch.Tensor, kind: str = "param") -> RaggedShardDTensor:
        """ya_fsdp/_param.py:298-310: wrap a local 1-D fragment of this parameter (same length as the sharded
        parameter's) with the parameter's sharding spec."""
        if tensor.shape != self._sharded_param_data.shape:
            raise AssertionError(f"Expects size {self._sharded_param_data.shape} but got {tensor.shape}")
        spec = self._sharding_spec
        if kind != spec.kind or tensor.dtype != spec.tensor_meta.dtype:
            spec = RaggedShardSpec(spec.mesh, spec.placements,
                                   TensorMeta(spec.tensor_meta.shape, spec.tensor_meta.stride, tensor.dtype), spec.owner, kind)
        return RaggedShardDTensor(tensor, spec, requires_grad=False)

    @property
    def _sharded_local_tensor(self) -> torch.Tensor:
        """ya_fsdp/_param.py:312-314."""
        return self.sharded_param._local_tensor

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
        new_local = local_tensor(new_param.detach())
        if new_local.data_ptr() != self._sharded_param_data.data_ptr() and self.sharded_numel > 0:
            from . import _native

            if new_local.device != self._sharded_param_data.device or new_local.numel() != self.sharded_numel:
                raise NotImplementedError(
                    "moving a sharded module to another device or changing its parameter sizes is not supported"
                )
            _native.flat_copy(self._sharded_param_data, new_local.contiguous().view(-1))
        self.sharded_param = nn.Parameter(
            self.to_sharded_dtensor(self._sharded_param_data), requires_grad=self.sharded_param.requires_grad
        )
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
