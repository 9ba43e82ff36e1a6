"""Parameter group: flat-buffer layout plus stream/event scheduling around the
buffer kernels (mirror of ya_fsdp/_param_group.py for the per-rank buffer path).

What is kept from the reference
  * one flat padded buffer per group, chunked evenly over the (logical) ranks so
    that shard boundaries fall mid-tensor (ya_fsdp/_param_group.py:245-406); the
    ragged split is computed in closed form (``_layout``) instead of with
    per-element index tensors;
  * shared, pre-allocated byte buffers that unsharded parameters and gradient
    accumulators are views into (:32-71, :409-457), two data buffers + one
    gradient buffer per shard group, sized by the largest sharing group
    (ya_fsdp/_state.py:200-288);
  * the owner / release-event hand-off of those buffers and the stream choice
    of unshard / reshard / post_backward / finalize_backward (:550-615, :655-791);
  * ``torch.profiler.record_function`` range names (:563, :669, :710, :740).

What differs
  * every tensor op on the path is a kernel launch through ``_collectives`` /
    ``_native``; the two foreach calls of post_backward are one launch with the
    pre-divide and the pad zero-fill fused in;
  * the side stream has the default priority (the reference asks for a
    high-priority stream, :80-88; mixed stream priorities are avoided on this
    platform);
  * DTensor wrapping, state-dict hooks and YCCL are outside this build: a group
    is constructed from a list of tensors (optionally with the modules that own
    them, so that sharded / unsharded views are swapped in on the modules).
"""

from __future__ import annotations

import weakref

import contextlib
import logging
import os
from enum import Enum, auto
from typing import Any, Generator, Sequence

import torch

from . import _native
from ._api import MixedPrecisionPolicy
from ._collectives import (
    MODE_ADD,
    MODE_COPY,
    MODE_SKIP,
    AllGatherResult,
    _get_gradient_divide_factors,
    all_gather,
    foreach_reduce_copy_in,
    reduce_scatter,
)
from ._common import FSDPMeshInfo, ShardedState, TrainingState, is_bw, profiler_range, resolve_device
from ._layout import ShardLayout, make_layout
from ._param import ParamModuleInfo, YaFSDPParam

logger = logging.getLogger("yafsdp_amd")


class YaFSDPBufferContext:
    """ya_fsdp/_param_group.py:32-71."""

    class BufferType(Enum):
        ALL_GATHER = auto()
        REDUCE_SCATTER = auto()

    def __init__(self, buffer_type: "YaFSDPBufferContext.BufferType"):
        self._buffer_type = buffer_type
        self.buffers: dict[torch.dtype | None, torch.Tensor] = {}
        self.yccl_handles: dict[torch.dtype | None, Any] = {}
        self.owner: YaFSDPParamGroup | None = None
        self.release_event: torch.cuda.Event | None = None

    def lazy_init(
        self,
        sizes_by_dtype: "dict[torch.dtype | None, int]",
        device: torch.device,
        yccl_handles: "dict[torch.dtype | None, Any] | None" = None,
    ) -> None:
        """Byte buffers allocated as bf16 and re-viewed, as at :53-69.  A communication handle registered for a
        dtype class owns that class's buffer (``add_all_gather_output_buffer`` / ``add_reduce_scatter_buffer``,
        each returning a bf16 tensor of the requested length).  All buffers start zero-filled so that pad lanes
        are defined from the first use on."""
        if yccl_handles is None:
            yccl_handles = dict.fromkeys(sizes_by_dtype)
        self.yccl_handles = yccl_handles
        buffer_method = {
            self.BufferType.ALL_GATHER: "add_all_gather_output_buffer",
            self.BufferType.REDUCE_SCATTER: "add_reduce_scatter_buffer",
        }[self._buffer_type]
        self.buffers = {}
        for dtype, size_in_bytes in sizes_by_dtype.items():
            numel = (size_in_bytes + 1) // torch.bfloat16.itemsize
            if (handle := yccl_handles.get(dtype)) is None:
                buffer = torch.zeros(numel, dtype=torch.bfloat16, device=device)
            else:
                buffer = getattr(handle, buffer_method)(numel)
                _check_handle_buffer(buffer, numel, device, buffer_method)
                if numel > 0:
                    _native.flat_fill(buffer, 0.0)
            self.buffers[dtype] = buffer.view(torch.uint8)
        self.owner = None
        self.release_event = None


def _check_handle_buffer(buffer: Any, numel: int, device: torch.device, method: str) -> None:
    if (
        not isinstance(buffer, torch.Tensor) or buffer.dtype != torch.bfloat16 or buffer.numel() != numel
        or buffer.device != device or not buffer.is_contiguous()
    ):
        raise TypeError(
            f"{method}({numel}) of the communication handle must return a contiguous bfloat16 tensor of {numel} "
            f"elements on {device}, got {type(buffer).__name__}"
            + (f" {buffer.dtype} {tuple(buffer.shape)} on {buffer.device}" if isinstance(buffer, torch.Tensor) else "")
        )


class YaFSDPCommContext:
    """ya_fsdp/_param_group.py:74-101."""

    def lazy_init(self, device: torch.device) -> None:
        self.device = device
        # one side stream serves both the all-gather and the reduce-scatter side (:85-88)
        self.all_gather_stream = torch.cuda.Stream(device=device)
        self.reduce_scatter_stream = self.all_gather_stream
        self.post_forward_order: list[YaFSDPParamGroup] = []

    def get_all_gather_stream(self, async_op: bool, training_state: TrainingState) -> torch.cuda.Stream:
        if not async_op and training_state in (TrainingState.FORWARD, TrainingState.PRE_BACKWARD):
            return self.all_gather_stream
        return torch.cuda.current_stream(self.device)


class YaFSDPParamGroup:
    """One group of parameters sharing flat buffers and collectives."""

    def __init__(
        self,
        params: Sequence[torch.Tensor],
        mesh_info: FSDPMeshInfo,
        device: torch.device,
        mp_policy: MixedPrecisionPolicy = MixedPrecisionPolicy(),
        shard_alignment: int = 8,
        names: Sequence[str] | None = None,
        module_fqn: str | None = None,
        modules: tuple = (),
    ):
        device = torch.device(device)
        if device.type != "cuda":
            raise RuntimeError(f"the buffer path runs on the GPU only, got device {device}")
        device = resolve_device(device)
        names = list(names) if names is not None else [f"param{i}" for i in range(len(params))]
        self.modules = tuple(modules)
        infos = _get_param_module_infos(list(params), self.modules) if self.modules else [None] * len(params)
        self.fsdp_params = [YaFSDPParam(p, mesh_info, device, n, mi) for p, n, mi in zip(params, names, infos)]
        self.mesh_info = mesh_info
        self.device = device
        self.mp_policy = mp_policy
        self.shard_alignment = int(shard_alignment)
        self._training_state = TrainingState.IDLE
        self._sharded_state = ShardedState.SHARDED
        self._module_fqn = module_fqn

        self.comm_ctx = YaFSDPCommContext()
        self._post_forward_indices: list[int] = []
        self.reduce_grads: bool = True
        self.reshard_after_forward: bool = True
        self.reshard_after_backward: bool = True
        self.gradient_divide_factor: float | None = None
        self.force_sum_reduction_for_comms: bool = False
        self.unshard_async_op: bool = False
        self.unshard_in_backward: bool = True
        # opt-in, not the reference's plan (ya_fsdp/_param_group.py:669-708 runs the foreach calls on the compute
        # stream): the reduce copy-in of a pass that reduces runs on the reduce-scatter stream as well, right in
        # front of the post-reduce, and the compute stream goes on with the next group's backward at once.
        # YAFSDP_REDUCE_COPY_IN_ON_SIDE_STREAM=1 turns it on for every group of a process whose code cannot change.
        self.reduce_copy_in_on_side_stream: bool = os.environ.get("YAFSDP_REDUCE_COPY_IN_ON_SIDE_STREAM", "0") == "1"
        self._all_gather_result: AllGatherResult | None = None
        self._post_reduce_event: torch.cuda.Event | None = None

        self._init_mp_dtypes()
        param_group_requires_grad = any(p.requires_grad for p in self.fsdp_params)
        self.data_buffer_ctx = YaFSDPBufferContext(YaFSDPBufferContext.BufferType.ALL_GATHER)
        self.grad_buffer_ctx = (
            YaFSDPBufferContext(YaFSDPBufferContext.BufferType.REDUCE_SCATTER) if param_group_requires_grad else None
        )
        # all-gather dtype classes (ya_fsdp/_param_group.py:194-227): key None holds the ordinary parameters, whose
        # all-gather dtype is the group's parameter dtype; every entry of the policy's all_gather_dtype_to_param_cls
        # holds the parameters that are instances of that tensor subclass.  Each class has flat buffers, a layout
        # and a table of its own; empty classes are dropped.
        cls_map = mp_policy.all_gather_dtype_to_param_cls or {}
        classes: dict[torch.dtype | None, list[YaFSDPParam]] = {
            None: [p for p in self.fsdp_params if not any(isinstance(p.param_data, c) for c in cls_map.values())]
        }
        for all_gather_dtype, param_cls in cls_map.items():
            classes[all_gather_dtype] = [p for p in self.fsdp_params if isinstance(p.param_data, param_cls)]
        self._all_gather_dtype_to_fsdp_params: dict[torch.dtype | None, list[YaFSDPParam]] = {
            dtype: params for dtype, params in classes.items() if params
        }
        if sum(map(len, self._all_gather_dtype_to_fsdp_params.values())) != len(self.fsdp_params):
            raise AssertionError("a parameter is an instance of more than one class of all_gather_dtype_to_param_cls")
        self._all_gather_input_set_dtypes: set[torch.dtype | None] = set()

        world_size, rank = mesh_info.shard_mesh_size, mesh_info.shard_mesh_rank
        self.layouts: dict[torch.dtype | None, ShardLayout] = {}
        self._unsharded_param_numels: dict[torch.dtype | None, list[int]] = {}
        self.padded_unsharded_param_numel: dict[torch.dtype | None, int] = {}
        self._padded_sharded_param_numel: dict[torch.dtype | None, int] = {}
        self._padded_sharded_param_data: dict[torch.dtype | None, torch.Tensor] = {}
        self._padded_sharded_param_grad: dict[torch.dtype | None, torch.Tensor | None] = {}
        self._sharded_param_numels: dict[torch.dtype | None, list[int]] = {}
        for all_gather_dtype, fsdp_params in self._all_gather_dtype_to_fsdp_params.items():
            numels = [p._orig_size.numel() for p in fsdp_params]
            layout = make_layout(numels, world_size, self.shard_alignment)  # :245-265
            self.layouts[all_gather_dtype] = layout
            self._unsharded_param_numels[all_gather_dtype] = numels
            self.padded_unsharded_param_numel[all_gather_dtype] = layout.padded_unsharded_numel
            self._padded_sharded_param_numel[all_gather_dtype] = layout.padded_sharded_numel
            shard = torch.zeros(layout.padded_sharded_numel, dtype=self.orig_dtype, device=device)
            self._padded_sharded_param_data[all_gather_dtype] = shard
            grad_shard = torch.zeros_like(shard) if param_group_requires_grad else None
            self._padded_sharded_param_grad[all_gather_dtype] = grad_shard
            sharded_numels = layout.sharded_numels(rank)  # :354-358, closed form
            global_offsets = layout.global_offsets(rank)  # :359-377
            per_rank = layout.per_rank_sharded_numels()  # :347-353
            self._sharded_param_numels[all_gather_dtype] = sharded_numels
            # flatten + shard (:300-339) without the full-size temporary: copy only the
            # fragment of each parameter that this rank owns
            pos = 0
            with torch.no_grad():
                for fsdp_param, n, go, sn in zip(fsdp_params, sharded_numels, global_offsets, per_rank):
                    frag = shard[pos : pos + n]
                    if n > 0:
                        src = fsdp_param.param_data.detach().view(-1)[go : go + n]
                        if type(src) is torch.Tensor:
                            _native.flat_copy(frag, src)
                        else:
                            # a tensor subclass: only its own dispatch knows how its values become a plain tensor
                            # (unsharded_param_data.copy_(fsdp_param.param_data.view(-1)), :324)
                            frag.copy_(src)
                    fsdp_param.init_sharded_param(
                        frag, grad_shard[pos : pos + n] if grad_shard is not None else None, global_offset=go,
                        shard_numels=sn,
                    )  # :379-406
                    pos += n
        for index, fsdp_param in enumerate(self.fsdp_params):
            fsdp_param._param_group_ref = weakref.ref(self)
            fsdp_param._index_in_group = index
        for all_gather_dtype, fsdp_params in self._all_gather_dtype_to_fsdp_params.items():
            for index, fsdp_param in enumerate(fsdp_params):
                fsdp_param._all_gather_class = all_gather_dtype
                fsdp_param._index_in_class = index
        self._tables: dict[torch.dtype | None, _native.TensorTable] = {}
        self._gather_tail_mb: int | None = None  # set_gather_tail_mb; None: the library's process-wide option
        # events that a kernel of the path records on its own dispatch (_native.launch_recording), kept per purpose:
        # each is only ever recorded on one stream, so a later record implies every earlier one
        self._completion_events: dict[Any, torch.cuda.Event] = {}
        # this rank's fragments of each class's gradient shard (built on first use, ya_fsdp/_collectives.py:191-214)
        self._fragment_tables: dict[torch.dtype | None, _native.TensorTable] = {}
        self._state_dict_hook_handles: list = []
        # version of the master shard at which a fused optimizer step last wrote the
        # all-gather input (None: never); see all_gather
        self._copy_in_shard_version: int | None = None
        # gradient norm fused into the post-reduce (optim.enable_fused_grad_norm): float64 buffer of partial sums and,
        # per all-gather dtype class, the class's slice of it and the version of the class's gradient shard those
        # sums describe (no entry / None: they describe nothing)
        self._grad_sumsq_partials: torch.Tensor | None = None
        self._grad_sumsq_slot: dict[Any, tuple[int, int]] = {}
        self._grad_sumsq_token: dict[Any, int | None] = {}

    # ------------------------------------------------------------ initialisation --
    def _init_mp_dtypes(self) -> None:
        """ya_fsdp/_param_group.py:459-485."""
        for fsdp_param in self.fsdp_params:
            fsdp_param.init_dtype_attrs(self.mp_policy)
        trainable = [p for p in self.fsdp_params if p.requires_grad]
        orig_dtypes = {p.orig_dtype for p in self.fsdp_params}
        param_dtypes = {p.param_dtype for p in self.fsdp_params}
        reduce_dtypes = {p.reduce_dtype for p in trainable}
        if len(orig_dtypes) != 1:
            raise AssertionError(f"YaFSDP expects uniform original parameter dtype but got {orig_dtypes}")
        self.orig_dtype = next(iter(orig_dtypes))
        if len(param_dtypes) != 1:
            raise AssertionError(f"YaFSDP expects uniform param dtype but got {param_dtypes}")
        self.param_dtype = next(iter(param_dtypes))
        if len(trainable) > 0 and len(reduce_dtypes) != 1:
            raise AssertionError(f"YaFSDP expects uniform reduce dtype but got {reduce_dtypes}")
        self.reduce_dtype = next(iter(reduce_dtypes)) if len(trainable) > 0 else None

    @property
    def all_gather_dtype(self) -> torch.dtype:
        return self.param_dtype or self.orig_dtype

    @property
    def reduce_scatter_dtype(self) -> torch.dtype:
        return self.reduce_dtype or self.param_dtype or self.orig_dtype

    def _ag_dtype(self, all_gather_dtype: torch.dtype | None) -> torch.dtype:
        """Element type of a class's all-gather input and gathered buffer (ya_fsdp/_param_group.py:420)."""
        return all_gather_dtype or self.param_dtype or self.orig_dtype

    # the default class (ordinary parameters), for callers that deal with one class only
    @property
    def has_extension_classes(self) -> bool:
        return any(dtype is not None for dtype in self._all_gather_dtype_to_fsdp_params)

    def _default_class(self, what: str) -> None:
        if None not in self._all_gather_dtype_to_fsdp_params:
            raise NotImplementedError(
                f"{what}: every parameter of {self} belongs to a tensor-subclass all-gather dtype class "
                f"({list(self._all_gather_dtype_to_fsdp_params)}); use the per-class dictionaries"
            )

    @property
    def layout(self) -> ShardLayout:
        self._default_class("layout")
        return self.layouts[None]

    def completion_event(self, purpose: Any) -> torch.cuda.Event:
        """The group's event for ``purpose`` (a hashable name), created on first use."""
        event = self._completion_events.get(purpose)
        if event is None:
            event = self._completion_events[purpose] = torch.cuda.Event()
        return event

    def set_gather_tail_mb(self, megabytes: int | None) -> None:
        """How many megabytes at the end of this group's reduce buffer the reduce copy-in stores write-through (they
        then sit in the memory-side cache when the post-reduce or the next group's reduce copy-in comes to the same
        buffer).  A store-policy choice that changes no result; None follows the library's process-wide option."""
        self._gather_tail_mb = megabytes
        for table in self._tables.values():
            table.set_option(_native.OPT_GATHER_TAIL_MB, -1 if megabytes is None else megabytes)

    @property
    def _table(self) -> "_native.TensorTable | None":
        return self._tables.get(None)

    @property
    def _fragment_table(self) -> "_native.TensorTable | None":
        return self._fragment_tables.get(None)

    def data_buffer_bytes_by_dtype(self) -> dict[torch.dtype | None, int]:
        """Bytes of the gathered buffer of every all-gather dtype class (ya_fsdp/_state.py:234-251)."""
        return {
            dtype: numel * self._ag_dtype(dtype).itemsize for dtype, numel in self.padded_unsharded_param_numel.items()
        }

    def grad_buffer_bytes_by_dtype(self) -> dict[torch.dtype | None, int]:
        """Bytes of the reduce buffer of every all-gather dtype class (ya_fsdp/_state.py:265-284)."""
        return {
            dtype: numel * self.reduce_scatter_dtype.itemsize
            for dtype, numel in self.padded_unsharded_param_numel.items()
        }

    def data_buffer_bytes(self) -> int:
        self._default_class("data_buffer_bytes")
        return self.data_buffer_bytes_by_dtype()[None]

    def grad_buffer_bytes(self) -> int:
        self._default_class("grad_buffer_bytes")
        return self.grad_buffer_bytes_by_dtype()[None]

    def _init_unsharded_params(self) -> None:
        """ya_fsdp/_param_group.py:409-457: typed views of the shared byte buffers,
        split into per-parameter views (the zero-copy copy-out)."""
        self._all_gather_output = {}
        self._reduce_scatter_input = {}
        data_bytes, grad_bytes = self.data_buffer_bytes_by_dtype(), self.grad_buffer_bytes_by_dtype()
        for all_gather_dtype, fsdp_params in self._all_gather_dtype_to_fsdp_params.items():
            layout = self.layouts[all_gather_dtype]
            t_pad, total = layout.padded_unsharded_numel, layout.total_numel
            numels = self._unsharded_param_numels[all_gather_dtype]
            ag = self.data_buffer_ctx.buffers[all_gather_dtype].narrow(0, 0, data_bytes[all_gather_dtype]).view(
                self._ag_dtype(all_gather_dtype)
            )
            self._all_gather_output[all_gather_dtype] = ag
            if self.grad_buffer_ctx is not None:
                rs = self.grad_buffer_ctx.buffers[all_gather_dtype].narrow(0, 0, grad_bytes[all_gather_dtype]).view(
                    self.reduce_scatter_dtype
                )
            else:
                rs = None
            self._reduce_scatter_input[all_gather_dtype] = rs
            assert ag.numel() == t_pad
            ag_views = ag[:total].split(numels)
            rs_views = rs[:total].split(numels) if rs is not None else (None,) * len(numels)
            for fsdp_param, v, g in zip(fsdp_params, ag_views, rs_views):
                fsdp_param.init_unsharded_param(v, g)

    def _validate_no_meta_params(self) -> None:
        """ya_fsdp/_param_group.py:939-951."""
        param_names_on_meta = [
            fsdp_param._param_fqn for fsdp_param in self.fsdp_params if fsdp_param.sharded_param.device.type == "meta"
        ]
        if param_names_on_meta:
            raise RuntimeError(
                "FSDP parameters should be materialized from meta device before training, "
                f"but the following were still on meta device: {param_names_on_meta}\n"
                "For example, call module.to_empty(device) to materialize to device and "
                "call module.reset_parameters() on each module to initialize values."
            )

    def lazy_init(self) -> None:
        """ya_fsdp/_param_group.py:487-547 (idempotent)."""
        if not hasattr(self.comm_ctx, "all_gather_stream"):
            self.comm_ctx.lazy_init(self.device)
        if any(dtype not in self.data_buffer_ctx.buffers for dtype in self._all_gather_dtype_to_fsdp_params):
            raise RuntimeError(
                "the data buffer of this group is not allocated: call init_shared_state(groups, device) first"
            )
        self._validate_no_meta_params()  # :491
        self._register_state_dict_hooks()  # :492
        self._init_unsharded_params()
        self._all_gather_input = {}
        self._reduce_scatter_output = {}
        for all_gather_dtype, fsdp_params in self._all_gather_dtype_to_fsdp_params.items():
            shard = self._padded_sharded_param_data[all_gather_dtype]
            sharded_numels = self._sharded_param_numels[all_gather_dtype]
            n_local = sum(sharded_numels)
            yccl_handle = self.data_buffer_ctx.yccl_handles.get(all_gather_dtype)
            if yccl_handle is not None:
                # the communication library owns the buffer it gathers from (:510-519)
                ag_dtype = self._ag_dtype(all_gather_dtype)
                if shard.numel() * ag_dtype.itemsize % torch.bfloat16.itemsize:
                    raise ValueError(
                        f"a communication handle exchanges bfloat16 elements, but the {ag_dtype} shard of {self} has "
                        f"{shard.numel()} elements: use an even shard_alignment"
                    )
                numel = shard.numel() * ag_dtype.itemsize // torch.bfloat16.itemsize
                buffer = yccl_handle.add_all_gather_input_buffer(numel)
                _check_handle_buffer(buffer, numel, self.device, "add_all_gather_input_buffer")
                if numel > 0:
                    _native.flat_fill(buffer, 0.0)
                ag_in = buffer.view(ag_dtype)
            elif all_gather_dtype is None and self.param_dtype is None:
                ag_in = shard  # :502-505
            else:
                ag_in = torch.zeros_like(shard, dtype=all_gather_dtype or self.param_dtype)  # :506-508
            self._all_gather_input[all_gather_dtype] = ag_in
            for fsdp_param, frag in zip(fsdp_params, ag_in[:n_local].split(sharded_numels)):
                fsdp_param.init_all_gather_input(frag)
            if self.grad_buffer_ctx is not None:
                rs = self._reduce_scatter_input[all_gather_dtype]
                s = self.layouts[all_gather_dtype].padded_sharded_numel
                r = self.mesh_info.shard_mesh_rank
                rs_out = rs[r * s : (r + 1) * s]  # chunk(W)[r], :531-535
                self._reduce_scatter_output[all_gather_dtype] = rs_out
                for fsdp_param, frag in zip(fsdp_params, rs_out[:n_local].split(sharded_numels)):
                    fsdp_param.init_reduce_scatter_output(frag)
            if all_gather_dtype not in self._tables:
                self._tables[all_gather_dtype] = _native.TensorTable(
                    self._unsharded_param_numels[all_gather_dtype],
                    self.layouts[all_gather_dtype].padded_unsharded_numel, self.device,
                )
                if self._gather_tail_mb is not None:
                    self._tables[all_gather_dtype].set_option(_native.OPT_GATHER_TAIL_MB, self._gather_tail_mb)

    # ------------------------------------------------------------------- runtime --
    @property
    def _all_gather_process_group(self) -> Any:
        return self.mesh_info.shard_process_group

    @property
    def _reduce_scatter_process_group(self) -> Any:
        return self.mesh_info.shard_process_group

    def unshard(self, async_op: bool = False) -> None:
        """ya_fsdp/_param_group.py:550-594."""
        if self._all_gather_result is not None:
            return
        if self.is_unsharded:
            return
        if not self.unshard_in_backward and self._training_state == TrainingState.PRE_BACKWARD:
            return
        logger.debug("%s", self._with_fqn(f"YaFSDP::{self._training_state.name.lower()}_unshard"))
        with profiler_range(self._with_fqn("YaFSDP::all_gather")):
            all_gather_stream = self.comm_ctx.get_all_gather_stream(async_op, self._training_state)
            data_buffer_ctx = self.data_buffer_ctx
            if (owner := data_buffer_ctx.owner) is not None and owner is not self:
                raise RuntimeError(f"{self} tried to acquire its data buffer, but it is in use by {owner}.")
            if (release_event := data_buffer_ctx.release_event) is not None:
                all_gather_stream.wait_event(release_event)
                data_buffer_ctx.release_event = None
            data_buffer_ctx.owner = self
            for all_gather_dtype, fsdp_params in self._all_gather_dtype_to_fsdp_params.items():
                self._all_gather_result = all_gather(
                    self,
                    fsdp_params,
                    self._padded_sharded_param_data[all_gather_dtype],
                    self._all_gather_input[all_gather_dtype],
                    self._all_gather_output[all_gather_dtype],
                    self._all_gather_process_group,
                    async_op,
                    all_gather_stream,
                    self.device,
                    self.param_dtype,
                    all_gather_dtype,
                    self.data_buffer_ctx.yccl_handles.get(all_gather_dtype),
                )

    def wait_for_unshard(self) -> AllGatherResult | None:
        """ya_fsdp/_param_group.py:596-602."""
        if (all_gather_result := self._all_gather_result) is None:
            return None
        all_gather_result.wait()
        self._to_unsharded()
        self._all_gather_result = None
        return all_gather_result

    def reshard(self) -> None:
        """ya_fsdp/_param_group.py:604-615."""
        if self._training_state == TrainingState.FORWARD and not self.reshard_after_forward:
            return
        logger.debug("%s", self._with_fqn(f"YaFSDP::{self._training_state.name.lower()}_reshard"))
        self._to_sharded()
        self.data_buffer_ctx.release_event = torch.cuda.current_stream(self.device).record_event()
        self.data_buffer_ctx.owner = None

    def pre_forward(self, module: Any = None, args: tuple = (), kwargs: dict | None = None):
        """ya_fsdp/_param_group.py:617-626.  Called without arguments it only
        unshards; with the hook arguments it also registers the post-backward
        hook on the inputs and returns ``(args, kwargs)``."""
        kwargs = {} if kwargs is None else kwargs
        with profiler_range(self._with_fqn("YaFSDP::pre_forward")):
            self._training_state = TrainingState.FORWARD
            self.unshard(self.unshard_async_op)
            self.wait_for_unshard()
            if module is not None:
                args, kwargs = self._register_post_backward_hook(args, kwargs)
            return args, kwargs

    def post_forward(self, module: Any = None, input: Any = None, output: Any = None) -> Any:
        """ya_fsdp/_param_group.py:628-635."""
        with profiler_range(self._with_fqn("YaFSDP::post_forward")):
            if not is_bw():
                self.reshard()
                self._record_post_forward()
            self._training_state = TrainingState.IDLE
            return output

    def _register_post_backward_hook(self, args: tuple, kwargs: dict) -> tuple[tuple, dict]:
        """ya_fsdp/_param_group.py:859-884: route the inputs that require
        gradients through an autograd node whose backward runs post_backward."""
        if not torch.is_grad_enabled():
            return args, kwargs
        from torch.utils._pytree import tree_flatten, tree_unflatten

        args_list, args_spec = tree_flatten(args)
        kwargs_list, kwargs_spec = tree_flatten(kwargs)
        flat = list(args_list) + list(kwargs_list)
        idx = [i for i, obj in enumerate(flat) if torch.is_tensor(obj) and obj.requires_grad]
        if not idx:
            return args, kwargs
        outs = RegisterPostBackwardFunction.apply(self, *[flat[i] for i in idx])
        for i, t in zip(idx, outs):
            flat[i] = t
        args = tree_unflatten(flat[: len(args_list)], args_spec)
        kwargs = tree_unflatten(flat[len(args_list) :], kwargs_spec)
        return args, kwargs

    def _record_post_forward(self) -> None:
        post_forward_index = len(self.comm_ctx.post_forward_order)
        self.comm_ctx.post_forward_order.append(self)
        self._post_forward_indices.append(post_forward_index)

    def pre_backward(self, default_prefetch: bool = True) -> None:
        """ya_fsdp/_param_group.py:644-653."""
        if self._training_state == TrainingState.PRE_BACKWARD:
            return
        with profiler_range(self._with_fqn("YaFSDP::pre_backward")):
            self._training_state = TrainingState.PRE_BACKWARD
            self.unshard(self.unshard_async_op)
            self.wait_for_unshard()
            if default_prefetch:
                self._backward_prefetch()

    def post_backward(self, *unused: Any) -> None:
        """ya_fsdp/_param_group.py:655-771.  Safe to call when the group took no part in the backward."""
        self._training_state = TrainingState.POST_BACKWARD
        compute_stream = torch.cuda.current_stream(self.device)
        # the stream that writes the reduce buffer: the compute stream as in the reference, or (opt-in, for a pass
        # that reduces) the reduce-scatter stream once the compute stream has produced this group's gradients
        on_side = self.reduce_copy_in_on_side_stream and self.reduce_grads and self.grad_buffer_ctx is not None
        current_stream = self.comm_ctx.reduce_scatter_stream if on_side else compute_stream
        if on_side:
            current_stream.wait_stream(compute_stream)
        if (grad_buffer_ctx := self.grad_buffer_ctx) is not None:
            if (owner := grad_buffer_ctx.owner) is not None and owner is not self:
                raise RuntimeError(f"{self} tried to acquire its gradient buffer, but it is in use by {owner}.")
            if (release_event := grad_buffer_ctx.release_event) is not None:
                current_stream.wait_event(release_event)
                grad_buffer_ctx.release_event = None
            grad_buffer_ctx.owner = self
        predivide_fused: dict[torch.dtype | None, bool] = {}
        copy_in_events: dict[torch.dtype | None, torch.cuda.Event] = {}
        reduced_in_one_launch = False
        with profiler_range(self._with_fqn("FSDP::post_backward_accumulate")), (
            torch.cuda.stream(current_stream) if on_side else contextlib.nullcontext()
        ):
            single_class = len(self._all_gather_dtype_to_fsdp_params) == 1
            for all_gather_dtype, fsdp_params in self._all_gather_dtype_to_fsdp_params.items():
                grads: list[torch.Tensor | None] = []
                modes: list[int] = []
                for fsdp_param in fsdp_params:
                    has_grad = fsdp_param.requires_grad and fsdp_param.unsharded_param.grad is not None
                    if has_grad and fsdp_param.unsharded_accumulated_grad is None:
                        grads.append(fsdp_param.unsharded_grad_data)
                        modes.append(MODE_COPY)  # _foreach_copy_, :693-700
                        fsdp_param.unsharded_param.grad = None
                        fsdp_param.unsharded_accumulated_grad = fsdp_param._unsharded_accumulated_grad
                    elif has_grad:
                        grads.append(fsdp_param.unsharded_grad_data)
                        modes.append(MODE_ADD)  # _foreach_add_, :701-708
                        fsdp_param.unsharded_param.grad = None
                    else:
                        grads.append(None)
                        modes.append(MODE_SKIP)
                if not any(m != MODE_SKIP for m in modes):
                    continue
                if on_side:
                    for grad in grads:  # allocated on the compute stream, read on this one
                        if grad is not None:
                            grad.record_stream(current_stream)
                assert grad_buffer_ctx is not None and all_gather_dtype in self._tables
                pre = None
                if self.reduce_grads:
                    pre, _, _, _ = _get_gradient_divide_factors(
                        self._reduce_scatter_process_group, self.reduce_scatter_dtype, self.gradient_divide_factor,
                        self.force_sum_reduction_for_comms,
                        yccl_handle=grad_buffer_ctx.yccl_handles.get(all_gather_dtype),
                    )
                    predivide_fused[all_gather_dtype] = True
                    if single_class and all_gather_dtype is None:
                        reduced_in_one_launch = self._reduce_in_one_launch(grads, modes, current_stream, on_side)
                if not reduced_in_one_launch and self.reduce_grads:
                    # the launch records its own completion: the reduce-scatter stream waits for that event instead
                    # of a marker placed behind the kernel in the compute stream's queue
                    copy_in_events[all_gather_dtype] = _native.launch_recording(
                        self.completion_event(("reduce_copy_in", all_gather_dtype, on_side)),
                        lambda: foreach_reduce_copy_in(
                            self, self._tables[all_gather_dtype], self._reduce_scatter_input[all_gather_dtype],
                            grads, modes, pre,
                        ),
                        current_stream,
                    )
                elif not reduced_in_one_launch:
                    foreach_reduce_copy_in(
                        self, self._tables[all_gather_dtype], self._reduce_scatter_input[all_gather_dtype], grads,
                        modes, pre,
                    )
        fsdp_params_with_grad_per_dtype: dict[torch.dtype | None, list[YaFSDPParam]] = {}
        with profiler_range(self._with_fqn("YaFSDP::post_backward_reshard")):
            if not self.reduce_grads:
                if self.reshard_after_backward:
                    self.reshard()
                return
            for all_gather_dtype, fsdp_params in self._all_gather_dtype_to_fsdp_params.items():
                fsdp_params_with_grad = []
                for fsdp_param in fsdp_params:
                    if fsdp_param.unsharded_accumulated_grad is not None:
                        fsdp_params_with_grad.append(fsdp_param)
                        fsdp_param.unsharded_accumulated_grad = None
                fsdp_params_with_grad_per_dtype[all_gather_dtype] = fsdp_params_with_grad
            if self.reshard_after_backward:
                self.reshard()
        if sum(map(len, fsdp_params_with_grad_per_dtype.values())) == 0:
            if grad_buffer_ctx is not None:
                grad_buffer_ctx.release_event = current_stream.record_event()
                grad_buffer_ctx.owner = None
            return
        assert grad_buffer_ctx is not None
        if reduced_in_one_launch:
            # the gradient shard is already written, on this stream (ya_fsdp/_collectives.py:216-217 for the rest)
            with profiler_range(self._with_fqn("YaFSDP::post_backward_reduce")):
                self._post_reduce_event = self.completion_event(("reduce_in_one_launch", on_side))  # recorded by that launch
                for fsdp_param in fsdp_params_with_grad_per_dtype[None]:
                    fsdp_param.sharded_param.grad = fsdp_param.sharded_param_grad
            grad_buffer_ctx.release_event = self._post_reduce_event
            grad_buffer_ctx.owner = None
            return
        with profiler_range(self._with_fqn("YaFSDP::post_backward_reduce")):
            for all_gather_dtype, fsdp_params in self._all_gather_dtype_to_fsdp_params.items():
                if not fsdp_params_with_grad_per_dtype[all_gather_dtype]:
                    continue  # nothing of this class took part in the pass: its reduce buffer holds no gradient
                self._post_reduce_event = reduce_scatter(
                    fsdp_params,
                    fsdp_params_with_grad_per_dtype[all_gather_dtype],
                    self._padded_sharded_param_grad[all_gather_dtype],
                    self._reduce_scatter_input[all_gather_dtype],
                    self._reduce_scatter_process_group,
                    self.comm_ctx.reduce_scatter_stream,
                    self.orig_dtype,
                    self.param_dtype,
                    self.reduce_dtype,
                    self.device,
                    self.gradient_divide_factor,
                    self.force_sum_reduction_for_comms,
                    self.mp_policy.bit32_acc_for_bit16_reduce_scatter,
                    grad_buffer_ctx.yccl_handles.get(all_gather_dtype),
                    predivide_fused=predivide_fused.get(all_gather_dtype, False),
                    ready_event=copy_in_events.get(all_gather_dtype),
                )
        grad_buffer_ctx.release_event = self._post_reduce_event
        grad_buffer_ctx.owner = None

    def _reduce_in_one_launch(self, grads: "list[torch.Tensor | None]", modes: "list[int]",
                              stream: "torch.cuda.Stream", on_side: bool = False) -> bool:
        """A shard group of size ONE whose gradients pass through the reduce buffer: the rank's chunk is the whole
        buffer and the "reduce-scatter" copies it onto itself (ya_fsdp/_collectives.py:140-150), so the reduce
        copy-in (ya_fsdp/_param_group.py:693-708), the divides (:139, :146-148, :165) and the copy or accumulation
        into the gradient shard (:185 / :189) run as one launch on the current stream, with the same rounding points
        and the same contents of the reduce buffer afterwards.  Returns False, having launched nothing, for every
        other case; the caller then takes the general route."""
        group = self._reduce_scatter_process_group
        if group.size() != 1 or self._grad_sumsq_slot:
            return False
        if list(self._all_gather_dtype_to_fsdp_params) != [None] or self._table is None:
            return False  # one launch per group: only for a group with the default class alone
        if self.grad_buffer_ctx is None or self.grad_buffer_ctx.yccl_handles.get(None) is not None:
            return False  # a communication handle owns the reduce: the general route calls it
        need = [p for p in self.fsdp_params if p.sharded_param.requires_grad]
        in_sharded = (
            (self.reduce_dtype is None and self.param_dtype is None) or self.reduce_dtype == self.orig_dtype
        ) and all(p.sharded_param.grad is None for p in need)  # ya_fsdp/_collectives.py:112-123
        if in_sharded:
            return False
        with_grad = [p for p in self.fsdp_params if p.unsharded_accumulated_grad is not None]
        if len(with_grad) != len(need):
            return False  # some fragments keep their old gradient: ya_fsdp/_collectives.py:191-214
        n_acc = sum(p.sharded_param.grad is not None for p in with_grad)
        if n_acc not in (0, len(with_grad)):
            return False
        pre, post, _, _ = _get_gradient_divide_factors(
            group, self.reduce_scatter_dtype, self.gradient_divide_factor, self.force_sum_reduction_for_comms
        )
        custom = (
            self.gradient_divide_factor
            if self.gradient_divide_factor is not None and pre is None and post is None
            else None
        )  # ya_fsdp/_collectives.py:141-145
        if custom is not None and (custom == 0 or custom != custom or abs(custom) == float("inf")):
            return False
        shard = self._padded_sharded_param_grad[None]
        if shard is None:
            return False
        if not _native.all_contiguous(grads):
            grads = [g if g is None or g.is_contiguous() else g.contiguous() for g in grads]
        self._grad_sumsq_token.pop(None, None)
        served = []
        _native.launch_recording(
            self.completion_event(("reduce_in_one_launch", on_side)),
            lambda: served.append(self._table.gather_in_post_reduce(
                grads, self._reduce_scatter_input[None], shard, n_acc > 0, modes,
                pre_factor=pre, post_factor=post, custom_divisor=custom,
            )),
            stream,
        )
        return bool(served and served[0])

    def _fragment_table_for(self, grad_shard: torch.Tensor, numels: "list[int]") -> "_native.TensorTable":
        """Table over one class's gradient shard whose tensors are this rank's fragments (for the mixed copy /
        accumulate case of ya_fsdp/_collectives.py:191-214); built on first use."""
        key = next(k for k, v in self._padded_sharded_param_grad.items() if v is grad_shard)
        table = self._fragment_tables.get(key)
        if table is None:
            table = self._fragment_tables[key] = _native.TensorTable(numels, grad_shard.numel(), grad_shard.device)
        return table

    def finalize_backward(self) -> None:
        """ya_fsdp/_param_group.py:773-783."""
        self._wait_for_post_backward()
        if self._all_gather_result is not None:
            self._all_gather_result.wait()
            self._all_gather_result = None
            self.data_buffer_ctx.owner = None
        self._post_forward_indices.clear()
        self._all_gather_input_set_dtypes.clear()
        self._training_state = TrainingState.IDLE

    def _wait_for_post_backward(self) -> None:
        """ya_fsdp/_param_group.py:785-791."""
        if self._post_reduce_event is not None:
            torch.cuda.current_stream(self.device).wait_event(self._post_reduce_event)
            self._post_reduce_event = None
            assert self.grad_buffer_ctx is not None
            assert self.grad_buffer_ctx.owner is None
            self.grad_buffer_ctx.release_event = None

    def _backward_prefetch(self) -> None:
        """ya_fsdp/_param_group.py:793-805."""
        if not self._post_forward_indices:
            return
        curr_index = self._post_forward_indices.pop()
        if (target_index := curr_index - 1) < 0:
            return
        target = self.comm_ctx.post_forward_order[target_index]
        if target.data_buffer_ctx is not self.data_buffer_ctx:
            self._prefetch_unshard(target, "backward")

    @staticmethod
    def _prefetch_unshard(target: "YaFSDPParamGroup", pass_type: str) -> None:
        """ya_fsdp/_param_group.py:807-827."""
        if pass_type == "backward":
            training_state = TrainingState.PRE_BACKWARD
        elif pass_type == "forward":
            training_state = TrainingState.FORWARD
        else:
            raise ValueError(f"Unknown pass type: {pass_type}")
        with profiler_range(f"YaFSDP::{pass_type}_prefetch for {target._module_fqn}"), target.use_training_state(
            training_state
        ):
            target.unshard(target.unshard_async_op)

    # ----------------------------------------------------- materialising copy-out --
    def copy_out_materialize(self, outs: Sequence[torch.Tensor | None]) -> None:
        """Copy the gathered flat buffer into separately allocated tensors (one
        launch).  The group's own unsharded parameters are zero-copy views
        (``_init_unsharded_params``); this is for consumers that need their own
        storage.  Runs on the current stream; call after ``wait_for_unshard``."""
        if self.has_extension_classes:
            raise NotImplementedError("copy_out_materialize serves groups with the default all-gather dtype class only")
        assert self._table is not None, "lazy_init() first"
        self._table.scatter_out(self._all_gather_output[None], [o.view(-1) if o is not None else None for o in outs])

    def _register_state_dict_hooks(self) -> None:
        """ya_fsdp/_param_group.py:886-909: ``state_dict()`` and ``load_state_dict()`` of a
        module that owns parameters of this group first put the sharded
        parameters back in place, so both see the fp32 shards whatever state the
        last forward left the group in."""
        if self._state_dict_hook_handles:
            return  # already registered
        modules_with_params = {p._module_info.module for p in self.fsdp_params if p._module_info is not None}

        def to_sharded_hook(*args: Any, **kwargs: Any) -> None:
            self._to_sharded()

        for module in modules_with_params:
            self._state_dict_hook_handles.append(module.register_state_dict_pre_hook(to_sharded_hook))
            self._state_dict_hook_handles.append(module._register_load_state_dict_pre_hook(to_sharded_hook))

    # ------------------------------------------------------------------ utilities --
    def _to_sharded(self) -> None:
        if not self.is_sharded:
            for fsdp_param in self.fsdp_params:
                fsdp_param.to_sharded()
            self._sharded_state = ShardedState.SHARDED

    def _to_unsharded(self) -> None:
        if not self.is_unsharded:
            for fsdp_param in self.fsdp_params:
                fsdp_param.to_unsharded()
            self._sharded_state = ShardedState.UNSHARDED

    @property
    def is_sharded(self) -> bool:
        return self._sharded_state == ShardedState.SHARDED

    @property
    def is_unsharded(self) -> bool:
        return self._sharded_state == ShardedState.UNSHARDED

    @contextlib.contextmanager
    def use_training_state(self, training_state: TrainingState) -> Generator[None, Any, None]:
        old = self._training_state
        self._training_state = training_state
        try:
            yield
        finally:
            self._training_state = old

    def _with_fqn(self, label: str) -> str:
        if self._module_fqn:
            return f"{label} ({self._module_fqn})"
        return label

    def __repr__(self) -> str:
        return f"YaFSDPParamGroup(fqn={self._module_fqn})"


def _get_param_module_infos(params: list, modules: tuple) -> list:
    """ya_fsdp/_param_group.py:942-968."""
    from torch.distributed.fsdp._common_utils import _named_parameters_with_duplicates

    params_set = {id(p) for p in params}
    info: dict[int, ParamModuleInfo] = {}
    for module in modules:
        for _, submodule in module.named_modules(remove_duplicate=False):
            for param_name, param in _named_parameters_with_duplicates(submodule, recurse=False):
                if id(param) in params_set:
                    if id(param) not in info:
                        info[id(param)] = ParamModuleInfo(submodule, param_name)
                    else:
                        info[id(param)].shared_modules.append(submodule)
                        info[id(param)].shared_param_names.append(param_name)
    if len(info) != len(params):
        raise AssertionError(f"Some parameters are not in the module tree of {modules}")
    return [info[id(p)] for p in params]


class RegisterPostBackwardFunction(torch.autograd.Function):
    """ya_fsdp/_param_group.py:971-992."""

    @staticmethod
    def forward(ctx: Any, param_group: YaFSDPParamGroup, *inputs: torch.Tensor):
        ctx.param_group = param_group
        return inputs

    @staticmethod
    def backward(ctx: Any, *grads: torch.Tensor):
        ctx.param_group.post_backward()
        return (None, *grads)


def init_shared_state(
    param_groups: Sequence[YaFSDPParamGroup], device: torch.device, num_data_buffers: int | None = 2,
    num_grad_buffers: int | None = 1, yccl_handle: Any | None = None,
) -> None:
    """Buffer assignment of ya_fsdp/_state.py:200-288 and :617-678 for groups
    that share one shard group: one communication context, ``num_data_buffers``
    data buffers handed out round-robin in group order, ``num_grad_buffers``
    gradient buffers; each buffer is as large as the largest group using it.
    ``None`` gives every group its own buffer.  ``yccl_handle``: a communication
    library object that owns all those buffers and performs the exchanges (see
    ``YaFSDPBufferContext.lazy_init``).  Ends with ``lazy_init`` of each group."""
    device = torch.device(device)
    if not param_groups:
        return
    comm_ctx = YaFSDPCommContext()
    comm_ctx.lazy_init(device)

    def assign(groups: Sequence[YaFSDPParamGroup], attr: str, count: int | None, size_of) -> None:
        if not groups:
            return
        n = len(groups) if count is None else min(count, len(groups))
        ctxs = [getattr(groups[i], attr) for i in range(n)]
        users: list[list[YaFSDPParamGroup]] = [[] for _ in range(n)]
        for i, g in enumerate(groups):
            users[i % n].append(g)
        for ctx, gs in zip(ctxs, users):
            sizes = [size_of(g) for g in gs]  # bytes per all-gather dtype class
            dtypes = {dtype for per_dtype in sizes for dtype in per_dtype}
            ctx.lazy_init({dtype: max(per_dtype.get(dtype, 0) for per_dtype in sizes) for dtype in dtypes}, device,
                          yccl_handles=dict.fromkeys(dtypes, yccl_handle))
            for g in gs:
                setattr(g, attr, ctx)

    assign(list(param_groups), "data_buffer_ctx", num_data_buffers, lambda g: g.data_buffer_bytes_by_dtype())
    assign(
        [g for g in param_groups if g.grad_buffer_ctx is not None], "grad_buffer_ctx", num_grad_buffers,
        lambda g: g.grad_buffer_bytes_by_dtype(),
    )
    for g in param_groups:
        g.comm_ctx = comm_ctx
        g.lazy_init()
