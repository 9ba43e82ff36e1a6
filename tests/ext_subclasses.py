"""Two small tensor subclasses with the all-gather extension hooks
(``fsdp_pre_all_gather`` / ``fsdp_post_all_gather``, ya_fsdp/_param.py:185-195,
210-217, 242-254, 281-291), shaped like the fp8 weight wrappers those hooks
exist for, with int8 in fp8's place so that every step has an exact integer
restatement:

* ``Int8Master``: what the model's parameter is before ``fully_shard`` and what
  the sharded parameter wraps afterwards: the fp32 master values.  Its
  ``fsdp_pre_all_gather`` quantises them to int8 with a fixed power-of-two step
  (the all-gather input, 1 byte per element) and hands the step on as metadata.
* ``Int8Weight``: what ``fsdp_post_all_gather`` builds around the gathered int8
  buffer: a tensor of the parameter's shape and compute dtype that dequantises
  when an op reads it.

Test infrastructure only.
"""

from __future__ import annotations

import torch

STEP = 2.0**-9  # quantisation step; a power of two, so dequantisation is exact in bf16 for |q| <= 127

aten = torch.ops.aten
# ops whose result is "the same tensor, seen differently": the result keeps the subclass
_STRUCTURAL = {
    aten.detach.default, aten.alias.default, aten.view.default, aten._unsafe_view.default, aten.reshape.default,
    aten.slice.Tensor, aten.t.default, aten.transpose.int, aten.clone.default, aten._to_copy.default,
    aten.new_zeros.default, aten.new_empty.default, aten.zeros_like.default, aten.empty_like.default,
}


def quantize(values: torch.Tensor) -> torch.Tensor:
    """fp32 -> int8 with the fixed step: round half to even, saturate at +-127."""
    return torch.clamp(torch.round(values.float() / STEP), -127, 127).to(torch.int8)


def dequantize(q: torch.Tensor, step: float, dtype: torch.dtype) -> torch.Tensor:
    return q.to(dtype) * step


class Int8Master(torch.Tensor):
    """Wrapper around the master values ``_data``; every op runs on them."""

    @staticmethod
    def __new__(cls, data: torch.Tensor) -> "Int8Master":
        return torch.Tensor._make_wrapper_subclass(
            cls, data.shape, strides=data.stride(), dtype=data.dtype, device=data.device, requires_grad=False
        )

    def __init__(self, data: torch.Tensor):
        self._data = data

    def __repr__(self) -> str:  # type: ignore[override]
        return f"Int8Master({self._data!r})"

    def __tensor_flatten__(self):
        return ["_data"], None

    @staticmethod
    def __tensor_unflatten__(inner_tensors, meta, outer_size, outer_stride):
        return Int8Master(inner_tensors["_data"])

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        kwargs = {} if kwargs is None else kwargs

        def unwrap(x):
            if isinstance(x, Int8Master):
                return x._data
            if isinstance(x, (list, tuple)):
                return type(x)(unwrap(y) for y in x)
            return x

        out = func(*unwrap(args), **{k: unwrap(v) for k, v in kwargs.items()})
        if func in _STRUCTURAL:
            return cls(out)
        if isinstance(out, torch.Tensor) and args and isinstance(args[0], Int8Master) and out is args[0]._data:
            return args[0]  # an in-place op returns what it was called on
        return out

    # ---- the all-gather extension -------------------------------------------------------------------------------
    def fsdp_pre_all_gather(self, mesh):
        return (quantize(self._data),), (STEP,)

    def fsdp_post_all_gather(self, all_gather_outputs, metadata, param_dtype, *, out=None):
        (q,) = all_gather_outputs
        step = metadata[0] if metadata is not None else None  # None: built before the first all-gather
        if out is not None:
            assert isinstance(out, Int8Weight), type(out)
            assert out._q.data_ptr() == q.data_ptr() and out._q.shape == q.shape
            out._step = step
            return None
        return Int8Weight(q, step, param_dtype), (q,)


class Int8Weight(torch.Tensor):
    """Compute-side view of a gathered int8 buffer: shape of ``q``, dtype ``dtype``; ops see ``q * step``."""

    @staticmethod
    def __new__(cls, q: torch.Tensor, step, dtype: torch.dtype) -> "Int8Weight":
        return torch.Tensor._make_wrapper_subclass(
            cls, q.shape, strides=q.stride(), dtype=dtype, device=q.device, requires_grad=False
        )

    def __init__(self, q: torch.Tensor, step, dtype: torch.dtype):
        self._q = q
        self._step = step

    def __repr__(self) -> str:  # type: ignore[override]
        return f"Int8Weight(step={self._step}, q={self._q!r})"

    def __tensor_flatten__(self):
        return ["_q"], (self._step, self.dtype)

    @staticmethod
    def __tensor_unflatten__(inner_tensors, meta, outer_size, outer_stride):
        return Int8Weight(inner_tensors["_q"], meta[0], meta[1])

    def dequantize(self) -> torch.Tensor:
        if self._step is None:
            raise RuntimeError("Int8Weight read before its first all-gather set the quantisation step")
        return dequantize(self._q, self._step, self.dtype)

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        kwargs = {} if kwargs is None else kwargs
        if func in (aten.detach.default, aten.alias.default, aten.t.default, aten.transpose.int, aten.view.default):
            w, *rest = args
            return Int8Weight(func(w._q, *rest, **kwargs), w._step, w.dtype)

        def unwrap(x):
            if isinstance(x, Int8Weight):
                return x.dequantize()
            if isinstance(x, (list, tuple)):
                return type(x)(unwrap(y) for y in x)
            return x

        return func(*unwrap(args), **{k: unwrap(v) for k, v in kwargs.items()})
