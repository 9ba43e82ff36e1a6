"""Per-parameter bookkeeping of a parameter group: every tensor here is a VIEW
into one of the group's flat buffers (mirror of ya_fsdp/_param.py, restricted to
what the buffer path touches).  The sharded parameter and its gradient are
``RaggedShardDTensor`` wrappers around 1-D views of the flat master / gradient
shard (ya_fsdp/_param.py:142-151).
"""

from __future__ import annotations

import weakref
from dataclasses import dataclass, field
from typing import Any

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


@dataclass
class ExtensionsData:
    """ya_fsdp/_param.py:35-41: what a tensor subclass's ``fsdp_pre_all_gather`` hands to its
    ``fsdp_post_all_gather``."""

    all_gather_metadata: Any | None = None

    def clear(self) -> None:
        self.all_gather_metadata = None


def _inner_tensor_names(t: torch.Tensor) -> "list[str] | None":
    """Attribute names of the inner tensors of a wrapper tensor subclass; None for a plain tensor."""
    if type(t) in (torch.Tensor, nn.Parameter) or not hasattr(t, "__tensor_flatten__"):
        return None
    return list(t.__tensor_flatten__()[0])


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
        self._sharded_param_data = sharded_param_data  # the plain fragment of the flat master shard
        # What the sharded parameter wraps (ya_fsdp/_param.py:145-152): for a plain parameter the fragment itself;
        # for a tensor subclass an instance of that subclass made by its own ``new_zeros``, whose first inner tensor
        # is then replaced by the fragment, so that the subclass's methods (the all-gather hooks among them) see the
        # master values of this rank.
        self._sharded_local: torch.Tensor = sharded_param_data
        if _inner_tensor_names(self.param_data) is not None:
            holder = self.param_data.detach().new_zeros(self.sharded_numel)
            if (holder_names := _inner_tensor_names(holder)) is None:
                raise AssertionError(
                    f"{type(self.param_data).__name__}.new_zeros returned a plain tensor: the subclass has to "
                    "return an instance of itself for the sharded parameter to keep its all-gather hooks"
                )
            inner = getattr(holder, holder_names[0])
            if inner.shape != sharded_param_data.shape or inner.dtype != sharded_param_data.dtype:
                raise AssertionError(
                    f"first inner tensor of {type(holder).__name__}.new_zeros({self.sharded_numel}) is "
                    f"{tuple(inner.shape)} {inner.dtype}, expected {tuple(sharded_param_data.shape)} "
                    f"{sharded_param_data.dtype}"
                )
            setattr(holder, holder_names[0], sharded_param_data)
            self._sharded_local = holder
        self._sharding_spec = RaggedShardSpec(  # :136-140 with the logical mesh in the DeviceMesh's place
            self.mesh_info, (self.placement,), TensorMeta(self._orig_size, self.param.stride(), self.param.dtype),
            weakref.ref(self), "param",
        )
        self.sharded_param = nn.Parameter(self.to_sharded_dtensor(self._sharded_local), requires_grad=self.requires_grad)
        self.sharded_param._yafsdp_param = weakref.ref(self)  # lets flat-shard optimizers find the owner
        if self.requires_grad:
            assert sharded_param_grad is not None
            self.sharded_param_grad = self.to_sharded_dtensor(sharded_param_grad, "grad")
        else:
            self.sharded_param_grad = None
        del self.param, self.param_data  # the group's flat shard now owns the values
        self._setattr_on_modules(self.sharded_param)
        self._init_extensions()

    def _init_extensions(self) -> None:
        """ya_fsdp/_param.py:185-195."""
        inner_tensor = self._sharded_local_tensor
        has_fsdp_pre_all_gather = hasattr(inner_tensor, "fsdp_pre_all_gather")
        has_fsdp_post_all_gather = hasattr(inner_tensor, "fsdp_post_all_gather")
        if has_fsdp_pre_all_gather != has_fsdp_post_all_gather:
            raise AssertionError(
                "Both fsdp_pre_all_gather and fsdp_post_all_gather should be defined "
                f"if using all-gather extensions: {inner_tensor}"
            )
        self._extensions_data = ExtensionsData() if has_fsdp_pre_all_gather else None

    @property
    def shard_mesh_from_root(self) -> FSDPMeshInfo:
        """What ``fsdp_pre_all_gather`` receives (ya_fsdp/_param.py:328-337 passes the shard ``DeviceMesh``): the
        logical shard mesh, i.e. its size and this rank."""
        return self.mesh_info

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
        """ya_fsdp/_param.py:203-231."""
        unsharded_tensor = all_gather_output.view(self._orig_size)  # zero-copy copy-out
        if self._extensions_data is not None:
            # the raw view is what to_unsharded() hands to the hook on every later unshard (:211-217); at this
            # point no all-gather has run and the metadata is still None, as in the reference
            self._all_gather_output = unsharded_tensor
            unsharded_tensor, _ = self._sharded_local_tensor.fsdp_post_all_gather(
                (unsharded_tensor,), self._extensions_data.all_gather_metadata, self.param_dtype or self.orig_dtype
            )
        self.unsharded_param = nn.Parameter(unsharded_tensor, requires_grad=self.requires_grad)
        self.unsharded_param._yafsdp_param = weakref.ref(self)
        if self.requires_grad:
            assert reduce_scatter_input is not None
            self._unsharded_accumulated_grad = reduce_scatter_input.view(self._orig_size)
        else:
            self._unsharded_accumulated_grad = None

    def set_all_gather_input(self) -> None:
        """ya_fsdp/_param.py:281-291: a tensor subclass with ``fsdp_pre_all_gather`` produces its own all-gather
        input (an fp8 cast, say) and the metadata its ``fsdp_post_all_gather`` will want; the input is copied into
        this parameter's fragment of the flat all-gather input.  Plain tensors have nothing to do."""
        if self.sharded_state != ShardedState.SHARDED:
            raise AssertionError(f"Expects to be in SHARDED, not {self.sharded_state}")
        if self._extensions_data is None:
            return
        all_gather_inputs, self._extensions_data.all_gather_metadata = self._sharded_local_tensor.fsdp_pre_all_gather(
            self.shard_mesh_from_root
        )
        (all_gather_input,) = all_gather_inputs
        dst = self._all_gather_input
        if all_gather_input.numel() != dst.numel():
            raise AssertionError(
                f"fsdp_pre_all_gather of {self._param_fqn} returned {all_gather_input.numel()} elements for a "
                f"fragment of {dst.numel()}"
            )
        if dst.numel() > 0:
            from . import _native

            _native.flat_copy(dst, all_gather_input.detach().contiguous().view(-1))

    def to_sharded(self) -> None:
        self._setattr_on_modules(self.sharded_param)
        self.sharded_state = ShardedState.SHARDED

    def to_unsharded(self) -> None:
        """ya_fsdp/_param.py:237-257."""
        if self._extensions_data is not None and self._extensions_data.all_gather_metadata is not None:
            # refresh what the subclass derives from this all-gather's metadata (quantisation scales, say) on the
            # existing unsharded tensor; its data already is the gathered buffer
            self._sharded_local_tensor.fsdp_post_all_gather(
                (self._all_gather_output,), self._extensions_data.all_gather_metadata,
                self.param_dtype or self.orig_dtype, out=self.unsharded_param,
            )
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
        if self._sharded_local is not self._sharded_param_data:
            # a tensor subclass: its own copy_ knows where the values go (self._sharded_param_data.copy_(...), :348)
            if new_local is not self._sharded_local and self.sharded_numel > 0:
                with torch.no_grad():
                    self._sharded_local.copy_(new_local)
        elif new_local.data_ptr() != self._sharded_param_data.data_ptr() and self.sharded_numel > 0:
            from . import _native

            if new_local.device != self._sharded_param_data.device or new_local.numel() != self.sharded_numel:
                raise NotImplementedError(
                    "moving a sharded module to another device or changing its parameter sizes is not supported"
                )
            _native.flat_copy(self._sharded_param_data, new_local.contiguous().view(-1))
        self.sharded_param = nn.Parameter(
            self.to_sharded_dtensor(self._sharded_local), requires_grad=self.sharded_param.requires_grad
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
