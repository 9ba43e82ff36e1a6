"""Per-module state machine of ``fully_shard`` (mirror of ya_fsdp/_state.py):
forward pre/post hooks, pre-backward tensor hooks, the root post-backward
callback, lazy initialisation of the shared communication context and buffers.
All host control flow; the bytes move in ``_param_group`` / ``_collectives``."""

from __future__ import annotations

import functools
import logging
import os
from typing import Any

import torch
import torch.nn as nn
from torch.autograd import Variable
from torch.distributed._composable_state import _get_module_state, _insert_module_state, _State
from torch.distributed.utils import _apply_to_tensors, _to_kwargs
from torch.utils._pytree import tree_flatten

from . import _native
from ._api import MixedPrecisionPolicy
from ._common import TrainingState, profiler_range
from ._param_group import YaFSDPCommContext, YaFSDPParamGroup

logger = logging.getLogger("yafsdp_amd")


class YaFSDPStateContext:
    """ya_fsdp/_state.py:39-53."""

    def __init__(self) -> None:
        self.all_states: list[YaFSDPState] = []
        self.iter_forward_root: YaFSDPState | None = None
        self.post_backward_final_callback_queued: bool = False
        self.is_last_backward: bool = True
        self.post_optim_event: torch.cuda.Event | None = None


def _cast_fp_tensor(dtype: torch.dtype, x: Any) -> Any:
    """ya_fsdp/_common.py:63-70."""
    if not isinstance(x, torch.Tensor) or not torch.is_floating_point(x) or x.dtype == dtype:
        return x
    return x.to(dtype)


class YaFSDPState(_State):
    def __init__(self) -> None:
        super().__init__()
        self._fsdp_param_group: YaFSDPParamGroup | None = None
        self._is_root: bool | None = None  # set during lazy init
        self._state_ctx = YaFSDPStateContext()
        self._comm_ctx = YaFSDPCommContext()
        self._training_state: TrainingState = TrainingState.IDLE
        self._states_to_forward_prefetch: list[YaFSDPState] = []
        self._states_to_backward_prefetch: list[YaFSDPState] = []
        self._auto_reshard_after_forward: bool | None = True
        self._modules_to_run_forward: set[nn.Module] = set()

    def init(self, modules: tuple, device: torch.device, mp_policy: MixedPrecisionPolicy,
             auto_reshard_after_forward: bool) -> None:
        """ya_fsdp/_state.py:72-101."""
        for module in modules:
            _insert_module_state(module, self)
        self._modules = modules
        self._device = device
        self._mp_policy = mp_policy
        self._auto_reshard_after_forward = auto_reshard_after_forward
        if len(modules) == 1:
            self._pre_forward_hook_handle = modules[0].register_forward_pre_hook(
                self._pre_forward, prepend=True, with_kwargs=True
            )
            self._post_forward_hook_handle = modules[0].register_forward_hook(self._post_forward, prepend=False)
        else:
            self._pre_forward_hook_handle = self._post_forward_hook_handle = self._register_group_forward_hooks()

    def _register_group_forward_hooks(self) -> list:
        """Several modules, one group (ya_fsdp/_state.py:575-613): the pre-forward
        logic runs before whichever module runs first in an iteration, the
        post-forward logic after the last of them has run."""
        pending = self._modules_to_run_forward
        members = set(self._modules)

        def pre_hook(module: nn.Module, args: tuple, kwargs: dict):
            if pending:
                return None
            pending.update(members)  # first of the group to run
            return self._pre_forward(module, args, kwargs)

        def post_hook_for(member: nn.Module):
            def post_hook(module: nn.Module, input: Any, output: Any):
                pending.discard(member)
                if pending:
                    return None
                return self._post_forward(module, input, output)

            return post_hook

        handles = [m.register_forward_pre_hook(pre_hook, prepend=True, with_kwargs=True) for m in self._modules]
        handles += [m.register_forward_hook(post_hook_for(m), prepend=False, always_call=True) for m in self._modules]
        return handles

    # ---------------------------------------------------------------- lazy init --
    def _root_pre_forward(self, module: nn.Module, args: tuple, kwargs: dict) -> tuple[tuple, dict]:
        """ya_fsdp/_state.py:103-125."""
        self._lazy_init()
        if self._state_ctx.iter_forward_root is not None:
            return args, kwargs
        self._state_ctx.iter_forward_root = self
        with profiler_range("YaFSDP::root_pre_forward"):
            if (event := self._state_ctx.post_optim_event) is not None:
                self._comm_ctx.all_gather_stream.wait_event(event)
                self._state_ctx.post_optim_event = None
            else:
                # wait for the optimizer step before the implicitly prefetched unshards
                self._comm_ctx.all_gather_stream.wait_stream(torch.cuda.current_stream(self._device))
            with profiler_range("YaFSDP::inputs_to_device"):
                args_tuple, kwargs_tuple = _to_kwargs(args, kwargs, self._device, False)
            args, kwargs = args_tuple[0], kwargs_tuple[0]
        return args, kwargs

    def _lazy_init(
        self,
        allow_no_grad_reduce: bool = False,
        param_group_to_data_buffer_ctx_idx: "dict[YaFSDPParamGroup, int] | None" = None,
        param_group_to_grad_buffer_ctx_idx: "dict[YaFSDPParamGroup, int] | None" = None,
        yccl_handle: Any | None = None,
        process_group_to_yccl_handle: "dict[Any, Any] | None" = None,
        data_buffer_ctx_idx_to_yccl_handle: "dict[int, Any] | None" = None,
        grad_buffer_ctx_idx_to_yccl_handle: "dict[int, Any] | None" = None,
    ) -> None:
        """ya_fsdp/_state.py:127-175.  ``allow_no_grad_reduce`` gives every group
        its own gradient buffer, which gradient accumulation without
        synchronisation needs (the unreduced gradients live in that buffer).
        The two maps replace the round-robin buffer assignment: group -> index
        (in module order) of the group whose buffer context it uses; as in the
        reference (:645-660) a map is only accepted where the default would give
        every group its own buffer.  The handle arguments name the communication
        library object (duck-typed: ``add_all_gather_input_buffer``,
        ``add_all_gather_output_buffer``, ``add_reduce_scatter_buffer``,
        ``all_gather``, ``reduce_scatter``, ``process_profiling_events``) that owns
        the buffers of a buffer context and performs its exchanges: one for all
        contexts, one per shard process group (here: per logical mesh), or one
        per buffer-context index (:663-677)."""
        if self._is_root is not None:
            return
        self._is_root = True
        if len(self._modules) > 1:
            raise RuntimeError(f"YaFSDP requires a single root module but got {self._modules}")  # ya_fsdp/_state.py:143-146
        root_module = self._modules[0]
        visited_states: set[YaFSDPState] = set()
        for module_name, module in root_module.named_modules():
            if (state := _get_module_fsdp_state(module)) is None:
                continue
            if module is not root_module:
                if state not in visited_states and state._is_root is not None:
                    raise RuntimeError(
                        "YaFSDP state has already been lazily initialized for "
                        f"{module_name}\nYaFSDP requires running forward through the root module first"
                    )
                state._is_root = False
            if state not in visited_states:
                self._state_ctx.all_states.append(state)
            visited_states.add(state)
        self._init_fqns()
        self._init_shared_state(allow_no_grad_reduce, param_group_to_data_buffer_ctx_idx,
                                param_group_to_grad_buffer_ctx_idx, yccl_handle, process_group_to_yccl_handle,
                                data_buffer_ctx_idx_to_yccl_handle, grad_buffer_ctx_idx_to_yccl_handle)
        self.validate_shared_state()
        for state in self._state_ctx.all_states:
            if state._fsdp_param_group:
                state._fsdp_param_group.lazy_init()

    def _init_shared_state(
        self,
        allow_no_grad_reduce: bool = False,
        param_group_to_data_buffer_ctx_idx: "dict[YaFSDPParamGroup, int] | None" = None,
        param_group_to_grad_buffer_ctx_idx: "dict[YaFSDPParamGroup, int] | None" = None,
        yccl_handle: Any | None = None,
        process_group_to_yccl_handle: "dict[Any, Any] | None" = None,
        data_buffer_ctx_idx_to_yccl_handle: "dict[int, Any] | None" = None,
        grad_buffer_ctx_idx_to_yccl_handle: "dict[int, Any] | None" = None,
    ) -> None:
        """ya_fsdp/_state.py:177-288 and :617-678: one communication context;
        two data buffers handed out round-robin in module order and one gradient
        buffer, each as large as the largest group that uses it; the last group on
        each data buffer keeps its parameters unsharded after forward."""
        self._comm_ctx.lazy_init(self._device)
        for state in self._state_ctx.all_states:
            state._state_ctx = self._state_ctx
            state._comm_ctx = self._comm_ctx
            if group := state._fsdp_param_group:
                group.comm_ctx = self._comm_ctx
        param_groups = [s._fsdp_param_group for s in self._state_ctx.all_states if s._fsdp_param_group is not None]
        if not param_groups:
            return
        no_reshard_after_forward = all(not g.reshard_after_forward for g in param_groups)

        def assign(groups, attr, count, size_of, ctx_idx=None, idx_to_handle=None):
            if not groups:
                return []
            if ctx_idx is not None:
                assert count is None  # ya_fsdp/_state.py:659-660
                ctxs, users, idxs = [], [], []
                for g in groups:  # buffer contexts in order of first use (:661-669)
                    ctx = getattr(groups[ctx_idx[g]], attr)
                    if not any(ctx is c for c in ctxs):
                        ctxs.append(ctx)
                        users.append([])
                        idxs.append(ctx_idx[g])
                    users[next(i for i, c in enumerate(ctxs) if c is ctx)].append(g)
            else:
                n = len(groups) if count is None else min(count, len(groups))
                ctxs = [getattr(groups[i], attr) for i in range(n)]
                users = [[] for _ in range(n)]
                idxs = list(range(n))
                for i, g in enumerate(groups):
                    users[i % n].append(g)
            for ctx, gs, idx in zip(ctxs, users, idxs):
                sizes = [size_of(g) for g in gs]  # bytes per all-gather dtype class (:234-251, :265-284)
                dtypes = {dtype for per_dtype in sizes for dtype in per_dtype}
                if idx_to_handle is not None:  # :668-677, in the reference's order of precedence
                    handle = idx_to_handle[idx]
                elif process_group_to_yccl_handle is not None:
                    handle = process_group_to_yccl_handle[gs[-1].mesh_info.shard_process_group]
                else:
                    handle = yccl_handle
                ctx.lazy_init({dtype: max(per_dtype.get(dtype, 0) for per_dtype in sizes) for dtype in dtypes},
                              self._device, yccl_handles=dict.fromkeys(dtypes, handle))
                for g in gs:
                    setattr(g, attr, ctx)
            return users

        data_users = assign(param_groups, "data_buffer_ctx", None if no_reshard_after_forward else 2,
                            lambda g: g.data_buffer_bytes_by_dtype(), param_group_to_data_buffer_ctx_idx,
                            data_buffer_ctx_idx_to_yccl_handle)
        for state_groups in data_users:
            last = state_groups[-1]
            owner_state = next(s for s in self._state_ctx.all_states if s._fsdp_param_group is last)
            if owner_state._auto_reshard_after_forward:
                last.reshard_after_forward = False  # ya_fsdp/_state.py:256-260
        grad_users = assign([g for g in param_groups if g.grad_buffer_ctx is not None], "grad_buffer_ctx",
                            None if allow_no_grad_reduce else 1, lambda g: g.grad_buffer_bytes_by_dtype(),
                            param_group_to_grad_buffer_ctx_idx, grad_buffer_ctx_idx_to_yccl_handle)
        # Which stores write through (and so stay in the 256-MB memory-side cache) depends on how soon the written
        # buffers come round again, and this is where that is known: the gradient buffers come round soonest (one
        # for all groups by default), and the written-through end of each survives until its next visit if all of
        # them fit that cache together (measured with 1, 2, 3 and 4 buffers in rotation: 128, 128, 85, 64 MB each).
        # The choice is made per group (its tables carry it), so two models in one process keep their own; the
        # process-wide options stay what the application set them to.
        policy = os.environ.get("YAFSDP_STORE_POLICY", "auto")
        if policy not in ("auto", "keep", *_native.STORE_POLICIES):
            raise ValueError(
                f"YAFSDP_STORE_POLICY={policy!r}: expected auto, keep or one of {sorted(_native.STORE_POLICIES)}"
            )
        if policy == "auto":
            tail_mb = min(128, 256 // max(1, len(grad_users)))
            for g in param_groups:
                g.set_gather_tail_mb(tail_mb if tail_mb >= 32 else 0)
        elif policy != "keep":
            _native.set_store_policy(policy)  # an explicit, process-wide choice of the application

    def validate_shared_state(self) -> None:
        """ya_fsdp/_state.py:290-414: enough buffers for overlap; at most one
        group per shared buffer may skip resharding / reducing; and two groups
        that are unsharded at the same time (a module and one of its
        descendants) must not share a buffer."""
        data_users: dict[Any, list[YaFSDPParamGroup]] = {}
        grad_users: dict[Any, list[YaFSDPParamGroup]] = {}
        for state in self._state_ctx.all_states:
            if (group := state._fsdp_param_group) is None:
                continue
            data_users.setdefault(group.data_buffer_ctx, []).append(group)
            if group.grad_buffer_ctx is not None:
                grad_users.setdefault(group.grad_buffer_ctx, []).append(group)
        num_groups = sum(map(len, data_users.values()))
        if len(data_users) < min(2, num_groups):
            raise ValueError(
                "num_data_buffers must be no less than min(2, num_param_groups)"
                f" for correct overlap, but got num_data_buffers={len(data_users)} num_param_groups={num_groups}."
            )
        for groups in data_users.values():
            if len(bad := [g for g in groups if not g.reshard_after_forward]) > 1:
                raise ValueError(
                    "Only one parameter group across groups which share a data buffer"
                    f" is allowed to have no reshard after forward, but got {bad}"
                )
            if len(bad := [g for g in groups if not g.reshard_after_backward]) > 1:
                raise ValueError(
                    "Only one parameter group across groups which share a data buffer"
                    f" is allowed to have no reshard after backward, but got {bad}"
                )
        for groups in grad_users.values():
            if len(bad := [g for g in groups if not g.reduce_grads]) > 1:
                raise ValueError(
                    "Only one parameter group across groups which share a grad buffer"
                    f" is allowed to have no grad reduce, but got {bad}"
                )
        data_ctx_prefix: dict[Any, str] = {}
        grad_ctx_prefix: dict[Any, str] = {}

        def validate_buffers(module: nn.Module, prefix: str = "") -> None:
            state = _get_module_fsdp_state(module)
            group = state._fsdp_param_group if state is not None else None
            if group is not None:
                if group.data_buffer_ctx in data_ctx_prefix:
                    raise RuntimeError(
                        f"Param groups of {prefix} and {data_ctx_prefix[group.data_buffer_ctx]} share a"
                        " data buffer, so they can't be unsharded at the same time."
                    )
                data_ctx_prefix[group.data_buffer_ctx] = prefix
                if group.grad_buffer_ctx is not None:
                    if group.grad_buffer_ctx in grad_ctx_prefix:
                        raise RuntimeError(
                            f"Param groups of {prefix} and {grad_ctx_prefix[group.grad_buffer_ctx]} share a"
                            " grad buffer, so they can't be unsharded at the same time."
                        )
                    grad_ctx_prefix[group.grad_buffer_ctx] = prefix
            for name, sub in module.named_children():
                validate_buffers(sub, prefix + ("." if prefix else "") + name)
            if group is not None:
                del data_ctx_prefix[group.data_buffer_ctx]
                if group.grad_buffer_ctx is not None:
                    del grad_ctx_prefix[group.grad_buffer_ctx]

        validate_buffers(self._modules[0])

    def _init_fqns(self) -> None:
        """ya_fsdp/_state.py:415-441."""
        root_module = self._modules[0]
        param_to_fsdp_param = {}
        module_to_group = {}
        for state in self._state_ctx.all_states:
            if group := state._fsdp_param_group:
                for fsdp_param in group.fsdp_params:
                    param_to_fsdp_param[fsdp_param.sharded_param] = fsdp_param
                for module in group.modules:
                    module_to_group[module] = group
        for param_name, param in root_module.named_parameters():
            if param in param_to_fsdp_param:
                param_to_fsdp_param[param]._param_fqn = param_name
        for module_name, module in root_module.named_modules():
            if module in module_to_group:
                group = module_to_group[module]
                group._module_fqn = module_name if group._module_fqn is None else f"{group._module_fqn}, {module_name}"

    # -------------------------------------------------------------------- hooks --
    # Order of events in one iteration, which is the reference's (ya_fsdp/_state.py:443-565): forward pre-hook
    # (root bookkeeping, input casts, the group's unshard, explicit prefetches) -> module forward -> forward
    # post-hook (the group's reshard, tensor hooks on the outputs) -> those tensor hooks during backward (the
    # group's unshard for backward, explicit prefetches) -> one callback at the end of backward that settles
    # every group.  A forward that runs INSIDE backward (activation recomputation) finds the state in
    # PRE_BACKWARD and passes through both forward hooks untouched.
    def _recomputing_in_backward(self) -> bool:
        return self._training_state == TrainingState.PRE_BACKWARD

    def _cast_floating_point(self, tree: Any, dtype: torch.dtype, label: str) -> Any:
        with profiler_range(label):
            return _apply_to_tensors(functools.partial(_cast_fp_tensor, dtype), tree)

    @staticmethod
    def _prefetch(states: "list[YaFSDPState]", phase: str) -> None:
        for other in states:
            if other._fsdp_param_group is not None:
                YaFSDPParamGroup._prefetch_unshard(other._fsdp_param_group, phase)

    def _pre_forward(self, module: nn.Module, args: tuple, kwargs: dict) -> tuple[tuple, dict]:
        if self._recomputing_in_backward():
            return args, kwargs
        self._training_state = TrainingState.FORWARD
        args, kwargs = self._root_pre_forward(module, args, kwargs)
        policy = self._mp_policy
        if policy.cast_forward_inputs and policy.param_dtype:
            args, kwargs = self._cast_floating_point((args, kwargs), policy.param_dtype, "YaFSDP::cast_forward_inputs")
        if self._fsdp_param_group:
            args, kwargs = self._fsdp_param_group.pre_forward(module, args, kwargs)
        self._prefetch(self._states_to_forward_prefetch, "forward")
        return args, kwargs

    def _post_forward(self, module: nn.Module, input: Any, output: Any) -> Any:
        if self._recomputing_in_backward():
            return output
        if self._fsdp_param_group:
            output = self._fsdp_param_group.post_forward(module, input, output)
        self._hook_outputs_for_backward(output)
        self._training_state = TrainingState.IDLE
        ctx = self._state_ctx
        if ctx.iter_forward_root is self:  # the outermost forward of this iteration has returned
            ctx.iter_forward_root = None
        if (dtype := self._mp_policy.output_dtype) is not None:
            output = self._cast_floating_point(output, dtype, "YaFSDP::cast_forward_outputs")
        return output

    def _hook_outputs_for_backward(self, output: Any) -> None:
        """Every output tensor that takes part in autograd announces this module's backward
        (ya_fsdp/_state.py:549-556); under ``no_grad`` there is no backward to announce."""
        if not torch.is_grad_enabled():
            return
        for leaf in tree_flatten(output)[0]:
            if torch.is_tensor(leaf) and leaf.requires_grad:
                leaf.register_hook(self._pre_backward)

    def _pre_backward(self, grad: torch.Tensor) -> torch.Tensor:
        self._training_state = TrainingState.PRE_BACKWARD
        self._queue_end_of_backward()
        explicit = self._states_to_backward_prefetch
        if self._fsdp_param_group:
            # without an explicit list the group prefetches its predecessor in forward order itself
            self._fsdp_param_group.pre_backward(not explicit)
        self._prefetch(explicit, "backward")
        return grad

    def _queue_end_of_backward(self) -> None:
        """The first module to enter backward queues the end-of-backward callback on the autograd engine, once
        per backward pass (ya_fsdp/_state.py:558-565)."""
        ctx = self._state_ctx
        if not ctx.post_backward_final_callback_queued:
            ctx.post_backward_final_callback_queued = True
            Variable._execution_engine.queue_callback(self._root_post_backward_final_callback)

    def _root_post_backward_final_callback(self) -> None:
        """End of a backward pass (ya_fsdp/_state.py:501-532): groups whose post-backward node never ran are
        reduced now, every state returns to IDLE, and after the last backward of an iteration the groups wait for
        their reductions and the recorded forward order is dropped."""
        ctx = self._state_ctx
        last = ctx.is_last_backward
        with profiler_range("YaFSDP::root_post_backward_callback"):
            for state in ctx.all_states:
                group = state._fsdp_param_group
                if group is not None and group._training_state != TrainingState.POST_BACKWARD:
                    group.post_backward()  # its forward inputs did not require gradient: no autograd node fired
                state._training_state = TrainingState.IDLE
                if group is not None:
                    group._training_state = TrainingState.IDLE
                if last:
                    state._finalize_backward()
                if group is not None:
                    _flush_profiling_events(group)
            if last:
                self._comm_ctx.post_forward_order.clear()
            ctx.post_backward_final_callback_queued = False

    def _finalize_backward(self) -> None:
        if self._modules_to_run_forward:  # ya_fsdp/_state.py:534-546
            logger.warning(
                "%d of the %d modules passed to fully_shard did not run forward before backward; pass only modules "
                "that run forward together. Modules that did not run forward: %s",
                len(self._modules_to_run_forward), len(self._modules), list(self._modules_to_run_forward),
            )
            self._modules_to_run_forward.clear()  # the next forward starts afresh
        if self._fsdp_param_group:
            self._fsdp_param_group.finalize_backward()


def _flush_profiling_events(group: YaFSDPParamGroup) -> None:
    """Communication-library handles attached to the group's buffers turn the events they recorded during the
    pass into profiler ranges (ya_fsdp/_state.py:517-529)."""
    for buffer_ctx in (group.data_buffer_ctx, group.grad_buffer_ctx):
        if buffer_ctx is None:
            continue
        for handle in buffer_ctx.yccl_handles.values():
            if handle is not None:
                handle.process_profiling_events()


def _get_module_fsdp_state(module: nn.Module) -> YaFSDPState | None:
    state = _get_module_state(module)
    return state if isinstance(state, YaFSDPState) else None
