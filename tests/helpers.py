"""Shared helpers for the parity tests."""

from __future__ import annotations

import numpy as np
import torch

INT_VIEW = {torch.float32: torch.int32, torch.bfloat16: torch.int16, torch.float16: torch.int16}
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def assert_bits_equal(a: torch.Tensor, b: torch.Tensor, what: str = "") -> None:
    """Bit-for-bit equality, except that any NaN matches any NaN (NaN payloads
    are not defined by the reference: its CPU vector cast and its scalar / GPU
    cast already disagree on them)."""
    assert a.dtype == b.dtype and a.shape == b.shape, (what, a.dtype, b.dtype, a.shape, b.shape)
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    if a.numel() == 0:
        return
    ai, bi = a.view(INT_VIEW[a.dtype]), b.view(INT_VIEW[b.dtype])
    if torch.equal(ai, bi):
        return
    nan_a, nan_b = torch.isnan(a), torch.isnan(b)
    bad = (ai != bi) & ~(nan_a & nan_b)
    if bad.any():
        idx = bad.view(-1).nonzero()[:5].view(-1).tolist()
        av, bv = a.view(-1), b.view(-1)
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {a.numel()} elements differ; first at {idx}: "
            f"{[av[i].item() for i in idx]} vs {[bv[i].item() for i in idx]}"
        )


def special_values_f32() -> torch.Tensor:
    """binary32 patterns that exercise rounding ties, subnormals, signed zeros,
    infinities and NaN in the casts to bf16 / fp16."""
    bits = [
        0x00000000, 0x80000000, 0x3F800000, 0xBF800000,
        0x3F808000, 0x3F818000, 0x3F808001, 0x3F807FFF, 0x3F80FFFF,  # bf16 ties / near ties
        0x7F7FFFFF, 0xFF7FFFFF, 0x7F7F8000, 0x7F7F7FFF,  # overflow to inf on rounding
        0x7F800000, 0xFF800000, 0x7FC00000, 0xFFC00001, 0x7F800001,  # inf / NaN
        0x00000001, 0x00008000, 0x00018000, 0x007FFFFF, 0x00800000, 0x80000001,  # fp32 subnormals
        0x38800000, 0x387FE000, 0x387FF000, 0x33000000, 0x33000001, 0x33800000,  # fp16 subnormal range
        0x477FE000, 0x477FEFFF, 0x477FF000, 0x47800000, 0x3C001000, 0x3C003000,  # fp16 overflow / ties
    ]
    return torch.from_numpy(np.array(bits, dtype=np.uint32).view(np.float32).copy())


def randn(gen: torch.Generator, n, std: float, dtype: torch.dtype) -> torch.Tensor:
    return (torch.randn(n, generator=gen, dtype=torch.float32) * std).to(dtype)


def mixed_values(gen: torch.Generator, n: int, dtype: torch.dtype, std: float = 0.02, specials: bool = True) -> torch.Tensor:
    """Seeded normal data with the special patterns spliced in at the front (``specials=False``: plain finite data)."""
    x = torch.randn(n, generator=gen, dtype=torch.float32) * std
    if not specials:
        return x.to(dtype)
    sp = special_values_f32()
    k = min(n, sp.numel())
    x[:k] = sp[:k]
    # a few wide-range values
    if n > k + 64:
        x[k : k + 64] = torch.randn(64, generator=gen) * torch.logspace(-45, 38, 64)
    return x.to(dtype)


def loc(t: torch.Tensor) -> torch.Tensor:
    """The local 1-D fragment behind a sharded parameter / gradient (a ``RaggedShardDTensor``); plain tensors as
    they are.  Detached, so that it can be compared and copied freely."""
    from yafsdp_amd._tensor import local_tensor

    return local_tensor(t.detach())
