"""Mixed-precision policy of a parameter group: the dtypes the buffer kernels convert between.

Field names, defaults and the one consistency rule are those of ya_fsdp/_api.py:6-22, because a policy object
written for the reference must construct and compare equal here.  What each field selects on this path:

``param_dtype``
    dtype of the data buffer and of the unsharded parameters; copy-in converts the master shard to it (round to
    nearest even) and copy-out hands out views or copies in it.  ``None`` keeps the masters' dtype.
``reduce_dtype``
    dtype of the reduce buffer that reduce copy-in fills.  ``None`` follows ``param_dtype``.
``output_dtype`` / ``cast_forward_inputs``
    casts of a wrapped module's floating-point outputs / inputs around forward; no buffer kernel is involved.
``bit32_acc_for_bit16_reduce_scatter``
    asks the exchange to accumulate a bfloat16 reduce buffer in 32 bits; on one GPU it is validated and carried.
``all_gather_dtype_to_param_cls``
    tensor-subclass parameters (for instance 8-bit weights) that gather in another dtype than they compute in:
    all-gather dtype -> parameter class, which gives such parameters a data buffer of their own per dtype.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class MixedPrecisionPolicy:
    param_dtype: torch.dtype | None = None
    reduce_dtype: torch.dtype | None = None
    output_dtype: torch.dtype | None = None
    cast_forward_inputs: bool = False
    bit32_acc_for_bit16_reduce_scatter: bool = False
    all_gather_dtype_to_param_cls: dict[torch.dtype, type] | None = None

    def __post_init__(self) -> None:
        wants_wide_accumulation = self.bit32_acc_for_bit16_reduce_scatter
        if wants_wide_accumulation and self.reduce_dtype != torch.bfloat16:
            # same message as the reference's, which callers may match on
            raise ValueError(
                f"bit32_acc_for_bit16_reduce_scatter requires reduce dtype to be bfloat16 , but got {self.reduce_dtype}."
            )
