"""Optimizer-side passes over the flat shards of ``fully_shard`` modules.

The reference runs gradient clipping and the optimizer as torch foreach ops
over the per-parameter fragments of each group's flat shard (the dispatch table
of its tensor subclass, ya_fsdp/_tensor.py:212-312; the legacy wrapper's
``clip_grad_norm_`` and ``zero_grad``, ya_fsdp/ya_fsdp.py:543-562, 591-601).
The fragments of one group are consecutive ranges of one buffer, so here each
of these is ONE kernel launch per group over the flat shard:

=============================================  ==============================
reference                                      here
=============================================  ==============================
``optimizer.zero_grad(set_to_none=False)``     ``zero_grad`` -> ``flat_fill``
``clip_grad_norm_`` (norms, coefficient,        ``clip_grad_norm_`` ->
``grad.mul_``)                                  ``flat_sumsq`` + ``clip_coef``
                                                + ``flat_scale``
``torch.optim.AdamW.step`` + next iteration's   ``FlatAdamW.step`` ->
copy-in cast (ya_fsdp/_collectives.py:53-54)    ``adamw_step``
=============================================  ==============================

There is no torch fallback: parameters must be float32 CUDA tensors.
"""

from __future__ import annotations

from typing import Any, Iterable, Sequence

import torch
import torch.nn as nn

from . import _native
from ._param import YaFSDPParam
from ._param_group import YaFSDPParamGroup
from ._tensor import local_tensor
from ._state import _get_module_fsdp_state

__all__ = ["FlatAdamW", "clip_grad_norm_", "grad_clip_coef", "zero_grad", "fsdp_param_groups",
           "enable_fused_grad_norm", "disable_fused_grad_norm"]


def fsdp_param_groups(modules: nn.Module | Iterable[nn.Module]) -> list[YaFSDPParamGroup]:
    """The parameter groups of every ``fully_shard`` module under ``modules``, in module order."""
    roots = [modules] if isinstance(modules, nn.Module) else list(modules)
    groups: list[YaFSDPParamGroup] = []
    seen: set[int] = set()
    for root in roots:
        for module in root.modules():
            state = _get_module_fsdp_state(module)
            group = state._fsdp_param_group if state is not None else None
            if group is not None and id(group) not in seen:
                seen.add(id(group))
                groups.append(group)
    return groups


def _grad_classes(modules: nn.Module | Iterable[nn.Module]) -> "list[tuple[YaFSDPParamGroup, Any]]":
    """Every flat gradient shard under ``modules``: one per parameter group and all-gather dtype class of it (key
    ``None``: the ordinary parameters; a dtype: the tensor-subclass parameters that are all-gathered in it,
    ya_fsdp/_param_group.py:194-227), in module order."""
    return [(g, key) for g in fsdp_param_groups(modules) for key, shard in g._padded_sharded_param_grad.items()
            if shard is not None]


def _owner(param: torch.Tensor) -> YaFSDPParam | None:
    ref = getattr(param, "_yafsdp_param", None)
    return ref() if ref is not None else None


def _merge(ranges: list[tuple[int, int]]) -> list[tuple[int, int]]:
    """Sorted half-open ranges with the adjacent ones joined."""
    out: list[tuple[int, int]] = []
    for lo, hi in sorted(r for r in ranges if r[1] > r[0]):
        if out and out[-1][1] == lo:
            out[-1] = (out[-1][0], hi)
        else:
            out.append((lo, hi))
    return out


def _fragment_offsets(group: YaFSDPParamGroup, key: Any = None) -> list[int]:
    offsets = [0]
    for n in group._sharded_param_numels[key]:
        offsets.append(offsets[-1] + n)
    return offsets


def _grad_ranges(group: YaFSDPParamGroup, indices: Sequence[int] | None = None, key: Any = None) -> list[tuple[int, int]]:
    """Ranges of one flat gradient shard of the group (class ``key``) that hold a gradient: the
    fragments of the parameters whose ``.grad`` is set (``indices``: positions in the class's parameter list).
    A gradient tensor that is not the group's own view (assigned by the user) is copied into it first.
    When every fragment has one, the range extends over the pad lanes (zeros)."""
    grad_shard = group._padded_sharded_param_grad[key]
    if grad_shard is None:
        return []
    fsdp_params = group._all_gather_dtype_to_fsdp_params[key]
    offsets = _fragment_offsets(group, key)
    ranges = []
    complete = indices is None or len(indices) == len(fsdp_params)
    for i in range(len(fsdp_params)) if indices is None else indices:
        fsdp_param = fsdp_params[i]
        grad = fsdp_param.sharded_param.grad if fsdp_param.requires_grad else None
        if grad is None:
            if offsets[i + 1] > offsets[i]:
                complete = False
            continue
        view = fsdp_param.sharded_param_grad
        grad_local, view_local = local_tensor(grad.detach()), view._local_tensor
        if grad_local.numel() and grad_local.data_ptr() != view_local.data_ptr():
            _native.flat_copy(view_local, grad_local.reshape(-1))
            fsdp_param.sharded_param.grad = view
        ranges.append((offsets[i], offsets[i + 1]))
    merged = _merge(ranges)
    if complete and merged == [(0, offsets[-1])]:
        return [(0, grad_shard.numel())]
    return merged


class _ClipState:
    """Per-device scratch of the norm computation: room for the partial sums of
    many buffers (grown on demand)."""

    _by_device: dict[torch.device, "_ClipState"] = {}

    def __init__(self, device: torch.device):
        self.device = device
        self.partials = torch.empty(16 * _native.SUMSQ_MAX_PARTIALS, dtype=torch.float64, device=device)

    @classmethod
    def get(cls, device: torch.device) -> "_ClipState":
        state = cls._by_device.get(device)
        if state is None:
            state = cls._by_device[device] = _ClipState(device)
        return state

    def reserve(self, n_buffers: int) -> torch.Tensor:
        need = n_buffers * _native.SUMSQ_MAX_PARTIALS
        if self.partials.numel() < need:
            self.partials = torch.empty(need, dtype=torch.float64, device=self.device)
        return self.partials


def enable_fused_grad_norm(modules: nn.Module | Iterable[nn.Module]) -> None:
    """From now on the post-reduce of every ``fully_shard`` group under
    ``modules`` (one per all-gather dtype class of the group) also leaves the
    partial sums of squares of the gradient shard it writes (``yafsdp_post_reduce_sumsq``), and ``grad_clip_coef`` /
    ``clip_grad_norm_`` over the same ``modules`` add those up instead of
    reading the shards again: 4 bytes per element less per step.  A group
    falls back to the read pass whenever its sums do not describe its current
    gradients: a parameter without a gradient, a torch op on a gradient since
    the reduce (seen through the shard's version counter), or one of this
    module's own passes that rewrites gradients (scaling, zero-fill).  Kernels
    launched on the gradient shard through ``_native`` directly are not seen."""
    classes = _grad_classes(modules)
    if not classes:
        raise ValueError("no fully_shard parameter group with gradients under the given modules")
    disable_fused_grad_norm(modules)
    device = classes[0][0].device
    slots, total = [], 0
    for g, key in classes:
        # one partial sum per tile of the post-reduce; the read pass that replaces it when the sums are stale writes
        # at least one per gradient range, and a class has at most as many ranges as parameters
        n_params = len(g._all_gather_dtype_to_fsdp_params[key])
        n = max(_native.post_reduce_sumsq_count(g._padded_sharded_param_grad[key].numel()), n_params, 1)
        slots.append((total, total + n))
        total += n
    partials = torch.zeros(total, dtype=torch.float64, device=device)
    for (g, key), slot in zip(classes, slots):
        g._grad_sumsq_partials = partials
        g._grad_sumsq_slot[key] = slot


def disable_fused_grad_norm(modules: nn.Module | Iterable[nn.Module]) -> None:
    for g in fsdp_param_groups(modules):
        g._grad_sumsq_partials = None
        g._grad_sumsq_slot.clear()
        g._grad_sumsq_token.clear()


def _fused_partials(classes: "Sequence[tuple[YaFSDPParamGroup, Any]]") -> torch.Tensor | None:
    """The shared buffer of partial sums if exactly these gradient shards fill it, slot after slot."""
    partials = classes[0][0]._grad_sumsq_partials
    if partials is None:
        return None
    end = 0
    for g, key in classes:
        slot = g._grad_sumsq_slot.get(key)
        if g._grad_sumsq_partials is not partials or slot is None or slot[0] != end:
            return None
        end = slot[1]
    return partials if end == partials.numel() else None


def grad_clip_coef(
    modules: nn.Module | Iterable[nn.Module], max_norm: float, norm_type: float = 2.0
) -> tuple[torch.Tensor, torch.Tensor]:
    """``(total_norm, clip_coef)`` as float32 device scalars, without touching
    the gradients: ``clip_coef = min(max_norm / (total_norm + 1e-6), 1)``
    (ya_fsdp/ya_fsdp.py:557-559).  Pass ``clip_coef`` to ``FlatAdamW.step`` to
    fuse the scaling into the optimizer pass.  One launch per gradient range
    plus one; no host synchronisation.  Calls on one device share a scratch
    buffer and must be ordered on one stream."""
    if norm_type not in (2, 2.0):
        raise NotImplementedError("only the 2-norm is implemented (ya_fsdp/ya_fsdp.py:544)")
    classes = _grad_classes(modules)
    if not classes:
        raise ValueError("no fully_shard parameter group with gradients under the given modules")
    groups = [g for g, _ in classes]
    device = groups[0].device
    norm_and_coef = torch.empty(2, dtype=torch.float32, device=device)
    fused = _fused_partials(classes)
    if fused is not None:
        # sums left by the post-reduce where they still describe the gradients; a read pass into the class's own
        # slot (zeroed first: it may write fewer sums than the slot holds) where they do not
        for g, key in classes:
            grad_shard = g._padded_sharded_param_grad[key]
            ranges = _grad_ranges(g, None, key)
            if ranges == [(0, grad_shard.numel())] and g._grad_sumsq_token.get(key) == grad_shard._version:
                continue
            lo, hi = g._grad_sumsq_slot[key]
            fused[lo:hi].zero_()
            pos = lo
            for k, (a, b) in enumerate(ranges):
                # leave one entry for each range still to come (the slot holds at least one per parameter)
                pos = _native.sumsq_partials(grad_shard[a:b], fused[: hi - (len(ranges) - 1 - k)], pos)
            g._grad_sumsq_token.pop(key, None)
        if fused.numel() > 4 * _native.SUMSQ_MAX_PARTIALS:  # long array: many workgroups first, then one
            scratch = _ClipState.get(device).reserve(1 + fused.numel() // (4096 * _native.SUMSQ_MAX_PARTIALS))
            count = _native.sumsq_reduce_partials(fused, fused.numel(), scratch)
            _native.clip_coef_from_partials(scratch, count, max_norm, norm_and_coef)
        else:
            _native.clip_coef_from_partials(fused, fused.numel(), max_norm, norm_and_coef)
        return norm_and_coef[0], norm_and_coef[1]
    work = [(g._padded_sharded_param_grad[key], lo, hi) for g, key in classes for lo, hi in _grad_ranges(g, None, key)]
    partials = _ClipState.get(device).reserve(max(len(work), 1))
    count = 0
    for grad_shard, lo, hi in work:
        count = _native.sumsq_partials(grad_shard[lo:hi], partials, count)
    _native.clip_coef_from_partials(partials, count, max_norm, norm_and_coef)
    return norm_and_coef[0], norm_and_coef[1]


def clip_grad_norm_(
    modules: nn.Module | Iterable[nn.Module], max_norm: float, norm_type: float = 2.0
) -> torch.Tensor:
    """Legacy ``YaFSDP.clip_grad_norm_`` (ya_fsdp/ya_fsdp.py:543-562) over the flat
    gradient shards of every group under ``modules``; returns the total norm.
    One read pass per group for the norm; the scaling pass costs no memory
    traffic when nothing is clipped (coefficient exactly 1)."""
    total_norm, coef = grad_clip_coef(modules, max_norm, norm_type)
    coef = coef.view(1)
    for group, key in _grad_classes(modules):
        grad_shard = group._padded_sharded_param_grad[key]
        group._grad_sumsq_token.pop(key, None)  # the gradients are rewritten
        for lo, hi in _grad_ranges(group, None, key):
            _native.flat_scale(grad_shard[lo:hi], coef)
    return total_norm


def zero_grad(modules: nn.Module | Iterable[nn.Module]) -> None:
    """``zero_grad(set_to_none=False)``: one fill per group over its flat gradient shard."""
    for group, key in _grad_classes(modules):
        group._grad_sumsq_token.pop(key, None)
        _native.flat_fill(group._padded_sharded_param_grad[key], 0.0)


class _Unit:
    """The parameters of one optimizer param group that live in one flat shard
    (an fsdp parameter group), or one plain tensor outside any group."""

    def __init__(self, group: YaFSDPParamGroup | None, params: list[torch.Tensor], indices: list[int], key: Any = None):
        self.group = group
        self.key = key  # all-gather dtype class of the group whose flat shard this is
        self.params = params
        self.indices = indices  # position of each parameter in the class's parameter list
        if group is not None:
            shard = group._padded_sharded_param_data[key]
            if shard.dtype != torch.float32:
                raise TypeError(f"FlatAdamW needs float32 master shards, got {shard.dtype} in {group}")
            self.numel = shard.numel()
            self.device = shard.device
        else:
            (p,) = params
            if p.dtype != torch.float32 or p.device.type != "cuda" or not p.is_contiguous():
                raise TypeError("FlatAdamW handles contiguous float32 CUDA parameters only")
            self.numel = p.numel()
            self.device = p.device
        self.exp_avg = torch.zeros(self.numel, dtype=torch.float32, device=self.device)
        self.exp_avg_sq = torch.zeros(self.numel, dtype=torch.float32, device=self.device)
        self.steps = [0] * len(params)

    def state_view(self, k: int, flat: torch.Tensor) -> torch.Tensor:
        """A range of a flat moment buffer as the optimizer state of parameter k: shaped like the parameter, i.e.
        wrapped like the sharded parameter itself (what ``torch.zeros_like(p)`` gives torch's own optimizers)."""
        p = self.params[k]
        if self.group is None:
            return flat.view(p.shape)
        return self.group._all_gather_dtype_to_fsdp_params[self.key][self.indices[k]].to_sharded_dtensor(flat, kind="")

    def fragment(self, k: int) -> tuple[int, int]:
        if self.group is None:
            return 0, self.numel
        offsets = _fragment_offsets(self.group, self.key)
        i = self.indices[k]
        return offsets[i], offsets[i + 1]


class FlatAdamW(torch.optim.Optimizer):
    """``torch.optim.AdamW`` (or ``Adam`` with ``decoupled_weight_decay=False``)
    for ``fully_shard`` modules: one fused launch per parameter group over its
    flat float32 shard (parameters, gradients and both moments are flat buffers
    of the shard's size), which also writes the 16-bit all-gather input of the
    next iteration, so that the copy-in cast of the next forward
    (ya_fsdp/_collectives.py:47-55) is already done.

    ``params`` is what ``torch.optim.AdamW`` takes (``model.parameters()`` after
    ``fully_shard``, or param-group dicts).  ``state[p]`` holds ``exp_avg`` /
    ``exp_avg_sq`` as views of the flat moment buffers, so ``state_dict()`` has
    the layout of torch's.  Operation order and rounding: see
    ``yafsdp_adamw_step`` in ``include/yafsdp_hip.h``."""

    def __init__(
        self,
        params: Iterable[torch.Tensor] | Iterable[dict[str, Any]],
        lr: float = 1e-3,
        betas: tuple[float, float] = (0.9, 0.999),
        eps: float = 1e-8,
        weight_decay: float = 1e-2,
        *,
        decoupled_weight_decay: bool = True,
        fuse_copy_in: bool = True,
    ):
        if not 0.0 <= float(lr):
            raise ValueError(f"Invalid learning rate: {lr}")
        if not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon value: {eps}")
        if not 0.0 <= betas[0] < 1.0 or not 0.0 <= betas[1] < 1.0:
            raise ValueError(f"Invalid beta parameters: {betas}")
        if not 0.0 <= weight_decay:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay,
                        decoupled_weight_decay=decoupled_weight_decay)
        super().__init__(params, defaults)
        self.fuse_copy_in = fuse_copy_in
        self._units: dict[int, list[_Unit]] = {}

    # ------------------------------------------------------------------ planning --
    def _units_of(self, pg_index: int, pg: dict[str, Any]) -> list[_Unit]:
        key = pg_index
        units = self._units.get(key)
        if units is not None and sum(len(u.params) for u in units) == len(pg["params"]):
            return units
        by_shard: dict[tuple[int, Any], tuple[YaFSDPParamGroup, Any, list[torch.Tensor], list[int]]] = {}
        units = []
        for p in pg["params"]:
            owner = _owner(p)
            group = owner._param_group_ref() if owner is not None else None
            if group is None:
                units.append(_Unit(None, [p], [0]))
                continue
            cls_key = owner._all_gather_class
            entry = by_shard.setdefault((id(group), cls_key), (group, cls_key, [], []))
            entry[2].append(p)
            entry[3].append(owner._index_in_class)
        for group, cls_key, ps, idx in by_shard.values():
            order = sorted(range(len(ps)), key=lambda k: idx[k])
            units.append(_Unit(group, [ps[k] for k in order], [idx[k] for k in order], cls_key))
        for unit in units:
            for k, p in enumerate(unit.params):
                lo, hi = unit.fragment(k)
                st = self.state[p]
                st["step"] = torch.tensor(0.0)
                st["exp_avg"] = unit.state_view(k, unit.exp_avg[lo:hi])
                st["exp_avg_sq"] = unit.state_view(k, unit.exp_avg_sq[lo:hi])
        self._units[key] = units
        return units

    # ---------------------------------------------------------------------- step --
    @torch.no_grad()
    def step(self, closure=None, *, grad_scale: torch.Tensor | None = None, zero_grad: bool = False):
        """One optimizer step.  ``grad_scale`` (one-element float32 device tensor,
        e.g. the coefficient from ``grad_clip_coef``) multiplies every gradient
        first, as a preceding ``grad.mul_`` would, without writing it back;
        ``zero_grad=True`` zero-fills the gradients in the same pass."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        if grad_scale is not None:
            grad_scale = grad_scale.view(1)
        for pg_index, pg in enumerate(self.param_groups):
            beta1, beta2 = pg["betas"]
            hyper = dict(lr=float(pg["lr"]), beta1=beta1, beta2=beta2, eps=pg["eps"],
                         weight_decay=pg["weight_decay"], decoupled=pg["decoupled_weight_decay"])
            for unit in self._units_of(pg_index, pg):
                self._step_unit(unit, hyper, grad_scale, zero_grad)
        return loss

    def _step_unit(self, unit: _Unit, hyper: dict[str, Any], grad_scale, zero_grad: bool) -> None:
        group = unit.group
        if group is None:
            (p,) = unit.params
            if p.grad is None:
                return
            unit.steps[0] += 1
            grad = p.grad
            if grad.dtype != torch.float32 or not grad.is_contiguous():
                raise TypeError("FlatAdamW needs contiguous float32 gradients")
            _native.adamw_step(p.view(-1), grad.view(-1), unit.exp_avg, unit.exp_avg_sq, None,
                               step=unit.steps[0], grad_scale=grad_scale, zero_grad=zero_grad, **hyper)
            return
        key = unit.key
        shard = group._padded_sharded_param_data[key]
        grad_shard = group._padded_sharded_param_grad[key]
        if grad_shard is None:
            return
        class_params = group._all_gather_dtype_to_fsdp_params[key]
        # launches: maximal runs of fragments that have a gradient and share a step count
        ranges = _grad_ranges(group, unit.indices, key)
        whole = ranges == [(0, shard.numel())]
        with_grad = [k for k, p in enumerate(unit.params) if p.grad is not None]
        if not with_grad:
            return
        for k in with_grad:
            unit.steps[k] += 1
        uniform = len({unit.steps[k] for k in with_grad}) == 1
        # the fused copy-in needs the whole shard rewritten in this pass; otherwise the
        # next forward casts the shard itself, as it does in the reference
        out16 = None
        # (a tensor-subclass class produces its all-gather input itself, through fsdp_pre_all_gather)
        if (self.fuse_copy_in and key is None and whole and uniform and len(unit.indices) == len(class_params)
                and group.param_dtype is not None and hasattr(group, "_all_gather_input") and group.is_sharded):
            out16 = group._all_gather_input[None]
        if whole and uniform:
            runs = [(0, shard.numel(), unit.steps[with_grad[0]])]
        else:
            runs = []
            for k in with_grad:
                lo, hi = unit.fragment(k)
                if hi > lo:
                    if runs and runs[-1][1] == lo and runs[-1][2] == unit.steps[k]:
                        runs[-1] = (runs[-1][0], hi, unit.steps[k])
                    else:
                        runs.append((lo, hi, unit.steps[k]))
        if zero_grad:
            group._grad_sumsq_token.pop(key, None)  # the gradients are rewritten
        for lo, hi, step in runs:
            _native.adamw_step(
                shard[lo:hi], grad_shard[lo:hi], unit.exp_avg[lo:hi], unit.exp_avg_sq[lo:hi],
                None if out16 is None else out16[lo:hi], step=step, grad_scale=grad_scale, zero_grad=zero_grad,
                **hyper,
            )
        if out16 is not None:
            # the next unshard finds its all-gather input ready (ya_fsdp/_collectives.py:47-55)
            for fsdp_param in class_params:
                fsdp_param.set_all_gather_input()
            group._all_gather_input_set_dtypes.add(None)
            group._copy_in_shard_version = shard._version

    # --------------------------------------------------------------- state dicts --
    def state_dict(self) -> dict[str, Any]:
        for units in self._units.values():
            for unit in units:
                for k, p in enumerate(unit.params):
                    self.state[p]["step"] = torch.tensor(float(unit.steps[k]))
        return super().state_dict()

    def load_state_dict(self, state_dict: dict[str, Any]) -> None:
        super().load_state_dict(state_dict)
        self._units.clear()
        loaded = {p: dict(st) for p, st in self.state.items()}
        for pg_index, pg in enumerate(self.param_groups):
            for unit in self._units_of(pg_index, pg):  # re-creates zeroed flat moments and their views
                for k, p in enumerate(unit.params):
                    st = loaded.get(p)
                    if not st:
                        continue
                    unit.steps[k] = int(float(st.get("step", 0)))
                    for name in ("exp_avg", "exp_avg_sq"):
                        src = local_tensor(st[name]) if name in st else None
                        if src is not None and src.numel():
                            _native.flat_copy(local_tensor(self.state[p][name]).view(-1),
                                              src.to(p.device, torch.float32).contiguous().view(-1))
                    self.state[p]["step"] = torch.tensor(float(unit.steps[k]))
