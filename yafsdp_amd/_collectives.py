"""Collective + buffer ops of one parameter group: the hot path.

Same function names, positional signatures and return types as
ya_fsdp/_collectives.py, so that the parameter-group code above it reads the
same.  Every tensor op of the reference on this path is replaced by one launch
of a gfx950 kernel through the C ABI (``_native``); there is no torch or CPU
fallback.

=====================================================  =========================
reference op                                           here
=====================================================  =========================
``all_gather_input.copy_(shard)`` (:53-54)             ``flat_copy_fanout`` (cast
``all_gather_output.copy_(all_gather_input)`` (:56-58)  and placement in one pass
                                                        over the shard), or
                                                        ``flat_copy`` each
``_div_if_needed(rs_input, pre)`` (:139)               fused into the reduce
                                                        copy-in launch, or
                                                        ``flat_div``
``output.copy_(rs_input [/ factor])`` (:140-150)       ``flat_copy`` /
                                                        ``flat_div_copy``
``_div_if_needed(output, post)`` + ``copy_``/``add_``   ``post_reduce``
(:165, :185, :189)
``_foreach_copy_`` + ``_foreach_add_`` (:191-214)       ``gather_in`` over the
                                                        chunk's fragments
=====================================================  =========================

One GPU: ``all_gather_group.size()`` may exceed 1 (logical world size).  The
inter-GPU exchange (:60-71, :152-164) is then reduced to this rank's share:
the all-gather writes this rank's slot of the gathered buffer, and the
reduce-scatter result is this rank's chunk with the division the collective
would have applied (``ReduceOp.AVG``: by the group size; pre-multiplied sum:
by the custom factor) applied as a post-divide in the same launch.
"""

from __future__ import annotations

import itertools

from typing import TYPE_CHECKING, Any, NamedTuple, Optional, Sequence

import torch

from . import _native

if TYPE_CHECKING:
    from ._param import YaFSDPParam
    from ._param_group import YaFSDPParamGroup

MODE_SKIP, MODE_COPY, MODE_ADD = _native.MODE_SKIP, _native.MODE_COPY, _native.MODE_ADD


class AllGatherResult(NamedTuple):
    """ya_fsdp/_collectives.py:20-28."""

    all_gather_event: torch.cuda.Event | None
    all_gather_work: Any | None

    def wait(self) -> None:
        if (event := self.all_gather_event) is not None:
            event.wait()
        if (work := self.all_gather_work) is not None:
            work.wait()


def all_gather(
    param_group: "YaFSDPParamGroup",
    fsdp_params: "list[YaFSDPParam]",
    padded_sharded_param_data: torch.Tensor,
    all_gather_input: torch.Tensor,
    all_gather_output: torch.Tensor,
    all_gather_group: Any,
    async_op: bool,
    all_gather_stream: torch.cuda.Stream,
    device: torch.device,
    param_dtype: torch.dtype | None,
    all_gather_dtype: torch.dtype | None,
    yccl_handle: Optional[Any],
) -> AllGatherResult:
    """ya_fsdp/_collectives.py:31-76.  ``yccl_handle``: a communication library that owns the all-gather input
    and the gathered buffer of this class and performs the exchange itself (``all_gather(input, output)`` on bf16
    views of both, :67-70); the copy-in into its input buffer stays here."""
    with torch.cuda.stream(all_gather_stream):
        if all_gather_dtype is None:
            if (
                (version := param_group._copy_in_shard_version) is not None
                and all_gather_dtype in param_group._all_gather_input_set_dtypes
                and padded_sharded_param_data._version != version
            ):
                # a fused optimizer step wrote the all-gather input, and a torch op has
                # changed the master shard since (load_state_dict, another optimizer):
                # the 16-bit copy is stale, cast again
                param_group._all_gather_input_set_dtypes.discard(all_gather_dtype)
            param_group._copy_in_shard_version = None
        world_size = all_gather_group.size()
        shard_numel = all_gather_input.numel()
        rank = all_gather_group.rank()
        slot = all_gather_output if world_size == 1 else all_gather_output[rank * shard_numel : (rank + 1) * shard_numel]
        placed = False
        all_gather_event = None

        def last(launch):
            """The final launch of this all-gather records the event that its consumers wait for."""
            nonlocal all_gather_event
            all_gather_event = _native.launch_recording(
                param_group.completion_event(("all_gather", all_gather_dtype)), launch, all_gather_stream
            )

        if all_gather_dtype not in param_group._all_gather_input_set_dtypes:
            for fsdp_param in fsdp_params:
                fsdp_param.set_all_gather_input()
            if all_gather_dtype is None and (param_dtype is not None or yccl_handle is not None):
                # copy-in: cast the master shard (:53-54; into a handle's buffer also without a cast, :50-52) and,
                # in the same pass over it, place the result where the all-gather would (:56-58, :60-65); the
                # version counter of the destination is untouched because no autograd op is involved
                if yccl_handle is not None and world_size > 1:
                    _native.flat_copy(all_gather_input, padded_sharded_param_data)  # the handle places it
                elif all(t.data_ptr() % 16 == 0 for t in (slot, all_gather_input, padded_sharded_param_data)):
                    last(lambda: _native.flat_copy_fanout([all_gather_input, slot], padded_sharded_param_data))
                    placed = True
                else:
                    _native.flat_copy(all_gather_input, padded_sharded_param_data)
            param_group._all_gather_input_set_dtypes.add(all_gather_dtype)
        if yccl_handle is not None and world_size > 1:
            yccl_handle.all_gather(all_gather_input.view(torch.bfloat16), all_gather_output.view(torch.bfloat16))  # :67-70
        elif not placed:
            # size-1 group (:56-58), or this rank's share of all_gather_into_tensor (:60-65)
            last(lambda: _native.flat_copy(slot, all_gather_input))
        all_gather_work = None
        if all_gather_event is None:
            all_gather_event = all_gather_stream.record_event()
    return AllGatherResult(all_gather_event, all_gather_work)


def sizes_to_slices(sizes: list[int]) -> list[slice]:
    """ya_fsdp/_collectives.py:79-90: consecutive slices of the given lengths.

    >>> sizes_to_slices([20, 20, 30])
    [slice(0, 20, None), slice(20, 40, None), slice(40, 70, None)]
    """
    ends = list(itertools.accumulate(sizes))
    return [slice(end - size, end) for size, end in zip(sizes, ends)]


def foreach_reduce_copy_in(
    param_group: "YaFSDPParamGroup",
    table: "_native.TensorTable",
    reduce_scatter_input: torch.Tensor,
    grads: Sequence[torch.Tensor | None],
    modes: Sequence[int],
    predivide_factor: float | None,
) -> None:
    """The two foreach calls of ya_fsdp/_param_group.py:693-708 as ONE launch:
    per parameter ``copy`` (first micro-batch), ``add`` (accumulation) or absent,
    with the pre-divide of ya_fsdp/_collectives.py:139 and the zero-fill of the
    pad lanes fused in.  Runs on the current (compute) stream, like the
    reference's foreach calls."""
    if not _native.all_contiguous(grads):
        # the reference's foreach ops accept strided gradients
        grads = [g if g is None or g.is_contiguous() else g.contiguous() for g in grads]
    table.gather_in(grads, reduce_scatter_input, modes, predivide_factor, zero_pad=True)


def reduce_scatter(
    fsdp_params: "list[YaFSDPParam]",
    fsdp_params_with_grad: "list[YaFSDPParam]",
    padded_sharded_param_grad: torch.Tensor,
    padded_unsharded_param_grad: torch.Tensor,
    reduce_scatter_group: Any,
    reduce_scatter_stream: torch.cuda.Stream,
    orig_dtype: torch.dtype,
    param_dtype: torch.dtype | None,
    reduce_dtype: torch.dtype | None,
    device: Any,
    gradient_divide_factor: float | None,
    force_sum_reduction_for_comms: bool,
    bit32_acc_for_bit16_reduce_scatter: bool,
    yccl_handle: Optional[Any],
    *,
    predivide_fused: bool = False,
    ready_event: "torch.cuda.Event | None" = None,
) -> torch.cuda.Event:
    """ya_fsdp/_collectives.py:93-218.

    ``predivide_fused``: the caller already applied the pre-divide inside the
    reduce copy-in launch (``foreach_reduce_copy_in``), so it is skipped here.
    ``ready_event``: recorded on the current stream when the reduce buffer was
    complete; the reduce-scatter stream then waits for it instead of for the
    whole current stream (:110-111).
    """
    # ``yccl_handle``: the communication library that owns the reduce buffer reduces it in place
    # (``reduce_scatter(buffer)`` on its bf16 view, :163-164: a sum, which is why the divide factors then put the
    # whole division after it, :229-230); this rank's chunk of the buffer holds the result afterwards.
    # bit32_acc_for_bit16_reduce_scatter only reaches the collective (acc_type=, :157-161) and is unused for a
    # group of size 1 (:140-150).  Here this rank's chunk is the only contribution to its reduce-scatter output,
    # and a binary32 sum of one 16-bit value rounds back to that value, so the flag changes nothing; the sum over
    # several contributions in binary32 is ``post_reduce_fanin``.
    if ready_event is not None:
        reduce_scatter_stream.wait_event(ready_event)
    else:
        reduce_scatter_stream.wait_stream(torch.cuda.current_stream(padded_sharded_param_grad.device))
    post_reduce_event = None
    with torch.cuda.stream(reduce_scatter_stream):
        world_size, rank = reduce_scatter_group.size(), reduce_scatter_group.rank()
        reduce_in_sharded = (
            ((reduce_dtype is None and param_dtype is None) or reduce_dtype == orig_dtype)
            and all(
                fsdp_param.sharded_param.grad is None
                for fsdp_param in fsdp_params
                if fsdp_param.sharded_param.requires_grad
            )
            and yccl_handle is None
        )  # :112-123
        shard_numel = padded_unsharded_param_grad.numel() // world_size
        chunk = padded_unsharded_param_grad[rank * shard_numel : (rank + 1) * shard_numel]  # :127-129
        predivide_factor, postdivide_factor, reduce_scatter_op, premul_scalar = _get_gradient_divide_factors(
            reduce_scatter_group,
            reduce_dtype or param_dtype or orig_dtype,
            gradient_divide_factor,
            force_sum_reduction_for_comms,
            yccl_handle=yccl_handle,
        )
        if not predivide_fused:
            _div_if_needed(padded_unsharded_param_grad, predivide_factor)  # :139
        if world_size == 1:
            custom = (
                gradient_divide_factor is not None and predivide_factor is None and postdivide_factor is None
            )  # :141-145
            output_tensor = padded_sharded_param_grad if reduce_in_sharded else chunk
            if custom:
                _native.flat_div_copy(output_tensor, padded_unsharded_param_grad, gradient_divide_factor)  # :146-148
            elif reduce_in_sharded:
                _native.flat_copy(output_tensor, padded_unsharded_param_grad)  # :150
            # else: output aliases the reduce buffer, copy_ onto itself is a no-op (:150)
            premul = None
        else:
            # this rank's share of reduce_scatter_tensor (:152-162): its chunk, scaled as the collective scales
            # every contribution.  AVG and the pre-multiplied sum are one op in the collective library
            # (ncclRedOpCreatePreMulSum; ncclAvg on floating-point data uses 1 / nRanks): the scalar is converted to
            # the data type and each contribution is multiplied by it, rounded, before the sum - a product with the
            # rounded reciprocal, not a division (they differ unless the factor is a power of two).
            if yccl_handle is not None:
                yccl_handle.reduce_scatter(padded_unsharded_param_grad.view(torch.bfloat16))  # :163-164
            if reduce_scatter_op == "AVG":
                premul = 1.0 / world_size
            elif reduce_scatter_op == "PREMUL_SUM":
                premul = premul_scalar  # 1 / gradient_divide_factor, :249
            else:
                premul = None
            output_tensor = chunk
        # post-divide (:165), or the collective's own scaling, fused with the copy / accumulate into the gradient
        # shard (:166-214); the reference never has both (a scaling collective comes with postdivide_factor None)
        post = postdivide_factor
        assert premul is None or post is None
        group_ref = getattr(fsdp_params[0], "_param_group_ref", None) if fsdp_params else None
        param_group = group_ref() if group_ref is not None else None
        # every parameter of the group gets a gradient in this pass: the whole shard is meaningful afterwards
        whole = len(fsdp_params_with_grad) == len(fsdp_params)
        cls_key = getattr(fsdp_params[0], "_all_gather_class", None) if fsdp_params else None
        if param_group is not None:
            param_group._grad_sumsq_token.pop(cls_key, None)
        if world_size > 1 and reduce_in_sharded:
            # the collective would have written straight into the shard (:124-125)
            post_reduce_event = _post_reduce(param_group, cls_key, whole, padded_sharded_param_grad, chunk, post,
                                             False, premul, reduce_scatter_stream)
        elif world_size == 1 and reduce_in_sharded:
            _div_if_needed(padded_sharded_param_grad, post)
        else:
            fsdp_params_which_require_grad = [p for p in fsdp_params if p.sharded_param.requires_grad]
            without_sharded_grad = [p for p in fsdp_params_with_grad if p.sharded_param.grad is None]
            with_sharded_grad = [p for p in fsdp_params_with_grad if p.sharded_param.grad is not None]
            if len(without_sharded_grad) == len(fsdp_params_which_require_grad):
                post_reduce_event = _post_reduce(param_group, cls_key, whole, padded_sharded_param_grad, output_tensor,
                                                 post, False, premul, reduce_scatter_stream)  # :185
            elif len(with_sharded_grad) == len(fsdp_params_which_require_grad):
                post_reduce_event = _post_reduce(param_group, cls_key, whole, padded_sharded_param_grad, output_tensor,
                                                 post, True, premul, reduce_scatter_stream)  # :189
            else:
                with_ids = {id(p) for p in with_sharded_grad}
                without_ids = {id(p) for p in without_sharded_grad}
                modes = [
                    MODE_ADD if id(p) in with_ids else (MODE_COPY if id(p) in without_ids else MODE_SKIP)
                    for p in fsdp_params
                ]
                numels = [p.sharded_numel for p in fsdp_params]
                if premul is not None:
                    _native.flat_premul(output_tensor, premul)  # the collective leaves its result in the chunk
                if param_group is None:
                    _native.post_reduce_fragments(padded_sharded_param_grad, output_tensor, numels, modes, post)
                else:
                    # :165 in place on the chunk, as the reference does it, then :191-214 as ONE launch whatever the
                    # pattern of modes: the chunk's fragments are the "tensors" of a table over the gradient shard
                    _div_if_needed(output_tensor, post)
                    table = param_group._fragment_table_for(padded_sharded_param_grad, numels)
                    fragments = list(output_tensor[: sum(numels)].split(numels))
                    table.gather_in(fragments, padded_sharded_param_grad, modes, None, zero_pad=False)
        if post_reduce_event is None:
            post_reduce_event = reduce_scatter_stream.record_event()
        for fsdp_param in fsdp_params_with_grad:
            fsdp_param.sharded_param.grad = fsdp_param.sharded_param_grad  # :216-217
        return post_reduce_event


def _post_reduce(
    param_group: "YaFSDPParamGroup | None", cls_key: Any, whole: bool, shard: torch.Tensor, chunk: torch.Tensor,
    post: float | None, accumulate: bool, premul: float | None = None, stream: "torch.cuda.Stream | None" = None,
) -> "torch.cuda.Event | None":
    """``post_reduce`` of one all-gather dtype class of a group; for a class
    with a slot for partial sums of squares (``optim.enable_fused_grad_norm``)
    and a pass that gives every parameter of it its gradient, the variant that
    also leaves the squared norm of the shard.  ``premul``: the scalar of a
    collective that scales inside the reduction (then there is no post-divide).
    Returns the event that the (one) launch recorded on its own dispatch, or
    None when the caller has to record one behind what was launched."""
    slot = param_group._grad_sumsq_slot.get(cls_key) if param_group is not None else None
    if slot is None or not whole:
        def launch():
            if premul is not None:
                _native.post_reduce_premul(shard, chunk, premul, accumulate)
            else:
                _native.post_reduce(shard, chunk, post, accumulate)

        if param_group is None or stream is None:
            launch()
            return None
        return _native.launch_recording(param_group.completion_event(("post_reduce", cls_key)), launch, stream)
    if premul is not None:
        _native.flat_premul(chunk, premul)
    lo, hi = slot
    end = _native.post_reduce_sumsq(shard, chunk, post, accumulate, param_group._grad_sumsq_partials[:hi], lo)
    if end < hi:  # the slot is added up as a whole: entries a read pass may have left beyond these sums go
        param_group._grad_sumsq_partials[end:hi].zero_()
    param_group._grad_sumsq_token[cls_key] = shard._version
    return None


def _get_gradient_divide_factors(
    reduce_scatter_group: Any,
    reduce_dtype: torch.dtype,
    factor: float | None,
    force_sum_reduction_for_comms: bool,
    yccl_handle: Optional[Any] = None,
) -> tuple[float | None, float | None, str, float | None]:
    """ya_fsdp/_collectives.py:221-267.  The reduce op is returned by name
    ("SUM", "AVG", "PREMUL_SUM") with the pre-multiplier as a fourth value,
    because no NCCL op object is needed on one GPU."""
    if yccl_handle is not None:
        force_sum_reduction_for_comms = True
    overflow_risk = reduce_dtype not in (torch.float32, torch.bfloat16)
    data_parallel_size = reduce_scatter_group.size()
    if not overflow_risk and not force_sum_reduction_for_comms:
        if factor is None:
            if data_parallel_size == 1:
                return None, None, "SUM", None
            return None, None, "AVG", None
        if factor == reduce_scatter_group.size():
            return None, None, "AVG", None
        return None, None, "PREMUL_SUM", 1 / factor
    if factor is None:
        factor = float(data_parallel_size)
    pre_factor: float | None
    if overflow_risk:
        pre_factor = 1
        while factor % pre_factor == 0 and factor / pre_factor > pre_factor:
            pre_factor *= 2
        post_factor = factor / pre_factor
    else:
        pre_factor, post_factor = None, factor
    return pre_factor, post_factor, "SUM", None


def _div_if_needed(tensor: torch.Tensor, div_factor: float | None) -> None:
    """ya_fsdp/_collectives.py:270-272."""
    if div_factor is not None and div_factor > 1:
        _native.flat_div(tensor, div_factor)
