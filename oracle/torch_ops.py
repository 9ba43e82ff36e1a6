"""The reference's torch-op sequence for the per-rank buffer path, on CPU tensors.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Every function performs
the same ops, in the same order and with the same in-place-ness, as the cited
reference lines, so every intermediate rounding is reproduced.  The one
departure, documented where it occurs: flat buffers start zero-filled so that
pad lanes (uninitialised ``torch.empty`` memory in the reference,
ya_fsdp/_param_group.py:53-59, 269-271, 281-283) have a defined value.
"""

from __future__ import annotations

from typing import Sequence

import torch


# --------------------------------------------------------------------------- #
# unshard side                                                                #
# --------------------------------------------------------------------------- #
def copy_in(all_gather_input: torch.Tensor, padded_sharded_param_data: torch.Tensor) -> None:
    """Copy-in: cast the master shard into the all-gather input
    (ya_fsdp/_collectives.py:53-54)."""
    all_gather_input.copy_(padded_sharded_param_data)


def extension_copy_in(param_all_gather_input: torch.Tensor, all_gather_input: torch.Tensor) -> None:
    """The per-parameter copy of a tensor subclass's all-gather input (what its
    ``fsdp_pre_all_gather`` returned) into the parameter's fragment of the flat
    all-gather input (ya_fsdp/_param.py:281-291)."""
    param_all_gather_input.copy_(all_gather_input)


def all_gather_single_rank(all_gather_output: torch.Tensor, all_gather_input: torch.Tensor) -> None:
    """The "all-gather" of a size-1 group (ya_fsdp/_collectives.py:56-58)."""
    all_gather_output.copy_(all_gather_input)


def unsharded_views(
    all_gather_output: torch.Tensor, numels: Sequence[int], sizes: Sequence[Sequence[int]]
) -> list[torch.Tensor]:
    """Zero-copy copy-out: unsharded parameters are views into the gathered
    buffer (ya_fsdp/_param_group.py:441-457, ya_fsdp/_param.py:209)."""
    numels = list(numels)
    return [
        v.view(tuple(sz))
        for v, sz in zip(all_gather_output[: sum(numels)].split(numels), sizes)
    ]


def copy_out_materialize(
    all_gather_output: torch.Tensor, numels: Sequence[int], outs: Sequence[torch.Tensor]
) -> None:
    """Materialising copy-out: the same split as ``unsharded_views`` followed by
    a ``copy_`` into separately allocated tensors."""
    numels = list(numels)
    for v, o in zip(all_gather_output[: sum(numels)].split(numels), outs):
        o.view(-1).copy_(v)


# --------------------------------------------------------------------------- #
# reduce side                                                                 #
# --------------------------------------------------------------------------- #
def reduce_copy_in(
    rs_views: Sequence[torch.Tensor], grads: Sequence[torch.Tensor], accumulate: bool
) -> None:
    """Flatten unsharded gradients into views of the reduce buffer: first
    micro-batch ``_foreach_copy_`` (ya_fsdp/_param_group.py:693-700), later ones
    ``_foreach_add_`` (ya_fsdp/_param_group.py:701-708)."""
    if len(rs_views) == 0:
        return
    if accumulate:
        torch._foreach_add_(list(rs_views), list(grads))
    else:
        torch._foreach_copy_(list(rs_views), list(grads))


def div_if_needed(tensor: torch.Tensor, div_factor: float | None) -> None:
    """ya_fsdp/_collectives.py:270-272 (note ``> 1``, not ``!= 1``)."""
    if div_factor is not None and div_factor > 1:
        tensor.div_(div_factor)


def get_gradient_divide_factors(
    world_size: int,
    reduce_dtype: torch.dtype,
    factor: float | None,
    force_sum_reduction_for_comms: bool,
    has_yccl_handle: bool = False,
) -> tuple[float | None, float | None, str, float | None]:
    """ya_fsdp/_collectives.py:221-267 with the process group reduced to its
    size.  Returns ``(pre, post, op, premul)`` where ``op`` is one of "SUM",
    "AVG", "PREMUL_SUM" and ``premul`` is the pre-multiplier of "PREMUL_SUM"."""
    if has_yccl_handle:
        force_sum_reduction_for_comms = True
    overflow_risk = reduce_dtype not in (torch.float32, torch.bfloat16)
    if not overflow_risk and not force_sum_reduction_for_comms:
        if factor is None:
            if world_size == 1:
                return None, None, "SUM", None
            return None, None, "AVG", None
        if factor == world_size:
            return None, None, "AVG", None
        return None, None, "PREMUL_SUM", 1 / factor
    if factor is None:
        factor = float(world_size)
    if overflow_risk:
        pre_factor: float | None = 1
        while factor % pre_factor == 0 and factor / pre_factor > pre_factor:
            pre_factor *= 2
        post_factor = factor / pre_factor
    else:
        pre_factor, post_factor = None, factor
    return pre_factor, post_factor, "SUM", None


def reduce_scatter_one_rank_share(
    output_tensor: torch.Tensor, op: str, world_size: int, premul: float | None = None
) -> None:
    """What ``dist.reduce_scatter_tensor(output, input, op=...)`` (ya_fsdp/_collectives.py:152-162) does to ONE
    rank's contribution, for the three ops ``_get_gradient_divide_factors`` can return (:243-249, 267), applied in
    place to this rank's chunk (the only contribution there is on one GPU).

    The arithmetic lives in the collective library (NCCL, RCCL on ROCm; a dependency of torch, not part of the
    reference's tree and not pinned by it).  Its published definition: ``ncclRedOpCreatePreMulSum(scalar)`` converts
    the scalar to the data type, multiplies every rank's input element by it and rounds the product to the data
    type *before* the sum; ``ncclAvg`` on floating-point data is that same op with the scalar ``1 / nRanks``
    (integers: sum, then divide); ``ncclSum`` leaves a single contribution as it is.  torch hands
    ``_make_nccl_premul_sum(1 / factor)`` over as that scalar cast to the tensor's dtype.  So neither op divides:
    for a group size or factor that is no power of two ``x * round(1 / f)`` differs from ``x / f``."""
    if op == "SUM":
        return
    if op == "AVG":
        scalar = 1.0 / world_size
    elif op == "PREMUL_SUM":
        assert premul is not None
        scalar = premul
    else:
        raise ValueError(op)
    # binary64 -> binary32 -> data type, then an elementwise product of two tensors of that type (computed in
    # binary32, where the product of two 16-bit values is exact, and rounded once to the data type)
    k = torch.tensor(scalar, dtype=torch.float64).to(torch.float32).to(output_tensor.dtype)
    output_tensor.mul_(torch.full_like(output_tensor, k.item()))


def reduce_scatter_local(
    padded_sharded_param_grad: torch.Tensor,
    padded_unsharded_param_grad: torch.Tensor,
    world_size: int,
    rank: int,
    predivide_factor: float | None,
    postdivide_factor: float | None,
    mode: str,
    sharded_numels: Sequence[int] | None = None,
    fragment_has_sharded_grad: Sequence[bool | None] | None = None,
    collective: "tuple[str, float | None] | None" = None,
) -> torch.Tensor:
    """ya_fsdp/_collectives.py:124-214 for the branch that goes through the
    reduce buffer (``reduce_in_sharded`` false), with the inter-GPU collective
    (ya_fsdp/_collectives.py:152-164) replaced by its one-rank share: the rank's
    chunk of the reduce buffer *is* the reduce-scatter result.

    ``mode``: "copy" (:185), "add" (:189) or "mixed" (:191-214).  For "mixed",
    ``fragment_has_sharded_grad[p]`` is True (accumulate), False (copy) or None
    (parameter produced no gradient: fragment untouched).  ``collective``: ``(op, premul)`` of the reduce-scatter
    (``reduce_scatter_one_rank_share``); None leaves the chunk as it is (a sum of one contribution)."""
    div_if_needed(padded_unsharded_param_grad, predivide_factor)  # :139
    output_tensor = padded_unsharded_param_grad.chunk(world_size)[rank]  # :127-129
    if collective is not None:
        reduce_scatter_one_rank_share(output_tensor, collective[0], world_size, collective[1])  # :152-162
    div_if_needed(output_tensor, postdivide_factor)  # :165
    if mode == "copy":
        padded_sharded_param_grad.copy_(output_tensor)  # :185
    elif mode == "add":
        padded_sharded_param_grad.add_(output_tensor)  # :189
    elif mode == "mixed":
        assert sharded_numels is not None and fragment_has_sharded_grad is not None
        sharded_numels = list(sharded_numels)
        n = sum(sharded_numels)
        grad_frags = padded_sharded_param_grad[:n].split(sharded_numels)
        out_frags = output_tensor[:n].split(sharded_numels)
        copy_idx = [i for i, f in enumerate(fragment_has_sharded_grad) if f is False]
        add_idx = [i for i, f in enumerate(fragment_has_sharded_grad) if f is True]
        if copy_idx:
            torch._foreach_copy_([grad_frags[i] for i in copy_idx], [out_frags[i] for i in copy_idx])
        if add_idx:
            torch._foreach_add_([grad_frags[i] for i in add_idx], [out_frags[i] for i in add_idx])
    else:
        raise ValueError(mode)
    return output_tensor


# ---------------------------------------------------------------------------
# optimizer-side passes over the flat shard (the reference forwards these torch
# ops to the local fragments, ya_fsdp/_tensor.py:212-312)
# ---------------------------------------------------------------------------
def clip_grad_norm_(grads: Sequence[torch.Tensor], max_norm: float) -> torch.Tensor:
    """Legacy ``YaFSDP.clip_grad_norm_`` (ya_fsdp/ya_fsdp.py:543-562) on one rank,
    norm_type 2: per-buffer norms in binary32, norm of the stack, squared, (the
    all-reduce over ranks is the identity here), root, coefficient, in-place
    scale.  Returns the total norm."""
    grad_norm = torch.linalg.vector_norm(
        torch.stack([torch.linalg.vector_norm(g.detach(), 2.0, dtype=torch.float32) for g in grads]),
        2.0,
        dtype=torch.float32,
    )
    total_norm = grad_norm**2.0
    total_norm = total_norm ** (1 / 2.0)
    total_norm_coef = max_norm / (total_norm + 1e-6)
    total_norm_coef = torch.clamp(total_norm_coef, max=1.0)
    for g in grads:
        g.mul_(total_norm_coef)
    return total_norm


def adam_step_torch_ops(
    param: torch.Tensor,
    grad: torch.Tensor,
    exp_avg: torch.Tensor,
    exp_avg_sq: torch.Tensor,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    eps: float,
    weight_decay: float,
    step: int,
    decoupled: bool = True,
) -> None:
    """The tensor ops of one torch.optim.Adam(W) step (torch/optim/adam.py,
    ``_single_tensor_adam``, non-capturable branch), in place."""
    if weight_decay != 0:
        if decoupled:
            param.mul_(1 - lr * weight_decay)
        else:
            grad = grad.add(param, alpha=weight_decay)
    exp_avg.lerp_(grad, 1 - beta1)
    exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    bias_correction1 = 1 - beta1**step
    bias_correction2 = 1 - beta2**step
    step_size = lr / bias_correction1
    bias_correction2_sqrt = bias_correction2**0.5
    denom = (exp_avg_sq.sqrt() / bias_correction2_sqrt).add_(eps)
    param.addcdiv_(exp_avg, denom, value=-step_size)


# ---------------------------------------------------------------------------
# legacy ``YaFSDP`` class (ya_fsdp/ya_fsdp.py, ya_fsdp/meta_param.py): the same
# flat-buffer ops under other names
# ---------------------------------------------------------------------------
def legacy_flatten_and_shard(params: Sequence[torch.Tensor], world_size: int, rank: int, yccl_padding: bool):
    """ya_fsdp/ya_fsdp.py:836-866: pad the total to a multiple of the world size (and the chunk to 8 elements
    with YCCL padding), concatenate the parameters and zeros, keep this rank's chunk.  Returns
    ``(padded_numel, shard)``."""
    total = sum(p.numel() for p in params)
    padded = total
    if padded % world_size != 0:
        padded += world_size - padded % world_size
    if yccl_padding:
        chunk = padded // world_size
        if chunk % 8 != 0:
            chunk += 8 - chunk % 8
            padded = chunk * world_size
    flat = torch.cat([p.reshape(-1) for p in params] + [torch.zeros(padded - total, dtype=params[0].dtype)])
    shard_size = padded // world_size
    return padded, flat.narrow(0, shard_size * rank, shard_size).clone()


def legacy_bit16_copy(bit16: torch.Tensor, master: torch.Tensor) -> None:
    """ya_fsdp/ya_fsdp.py:519-520: ``_main_parameter_bit16.data.copy_(_main_parameter)``."""
    bit16.copy_(master)


def legacy_grad_buffer_upcast(fp32_buffer: torch.Tensor, grad_buffer: torch.Tensor) -> None:
    """ya_fsdp/ya_fsdp.py:945-954: ``reusable_fp32_grad_buffer.get().copy_(grad_reusable_buffer.get())``."""
    fp32_buffer.copy_(grad_buffer)


def legacy_accumulate_shard(fp32_grad_shard: torch.Tensor, target: torch.Tensor) -> None:
    """ya_fsdp/ya_fsdp.py:991-992: ``self.fp32_grad_shard.add_(target_tensor)``."""
    fp32_grad_shard.add_(target)


def legacy_final_divide(grad: torch.Tensor, world_size: int, accumulation_steps: int) -> None:
    """ya_fsdp/ya_fsdp.py:499-501: ``grad.data.div_(world_size * gradient_accumulation_steps)``."""
    grad.div_(world_size * accumulation_steps)


def legacy_narrow_backward(grad_buffer: torch.Tensor, offset: int, grad_output: torch.Tensor, accumulate: bool) -> None:
    """ya_fsdp/meta_param.py:16-27: the per-parameter gradient lands in its range of the flat gradient buffer,
    ``copy_`` on the first micro-batch and ``add_`` afterwards."""
    view = grad_buffer.narrow(0, offset, grad_output.numel())
    if not accumulate:
        view.copy_(grad_output.reshape(-1))
    else:
        view.add_(grad_output.reshape(-1))


# ---------------------------------------------------------------------------
# the two exchange points over several buffers (one GPU: all local)
# ---------------------------------------------------------------------------
def copy_in_fanout(dsts: Sequence[torch.Tensor], padded_sharded_param_data: torch.Tensor) -> None:
    """The copy-in cast (ya_fsdp/_collectives.py:53-54) landing in this rank's slot of
    several gathered buffers, which is where ``all_gather_into_tensor`` puts it
    (:60-65)."""
    for d in dsts:
        d.copy_(padded_sharded_param_data)


def reduce_scatter_fanin(
    padded_sharded_param_grad: torch.Tensor,
    chunks: Sequence[torch.Tensor],
    postdivide_factor: float | None,
    accumulate: bool,
    premul: float | None = None,
) -> None:
    """A reduce-scatter over the ranks' chunks with binary32 accumulation in rank
    order (``acc_type=torch.float32``, ya_fsdp/_collectives.py:157-161) whose output
    has the reduce dtype, then the post-divide (:165) and ``copy_`` / ``add_``
    into the gradient shard (:185 / :189).  ``premul``: the collective scales
    inside the reduction (``ReduceOp.AVG`` = 1 / ranks, or ``_make_nccl_premul_sum``,
    :243-249) - the collective library converts the scalar to the data type and
    multiplies every rank's element by it in that type before the sum."""
    dtype = chunks[0].dtype
    if premul is not None:
        assert postdivide_factor is None
        scalar = torch.tensor(premul, dtype=torch.float32).to(dtype)
        chunks = [c * scalar for c in chunks]  # same-dtype tensor product: rounds to dtype
    acc = chunks[0].to(torch.float32).clone()
    for c in chunks[1:]:
        acc.add_(c.to(torch.float32))
    output_tensor = acc.to(dtype)
    div_if_needed(output_tensor, postdivide_factor)
    if accumulate:
        padded_sharded_param_grad.add_(output_tensor)
    else:
        padded_sharded_param_grad.copy_(output_tensor)
