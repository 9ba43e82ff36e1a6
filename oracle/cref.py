"""ctypes loader for the plain-C restatement: TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os

import numpy as np
import torch

from . import build as _build

DT = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = _build.OUT
        if not os.path.exists(path):
            path = _build.build()
        L = ctypes.CDLL(path)
        vp, i64, dbl, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_double, ctypes.c_int
        L.ref_f32_to_bf16.restype = ctypes.c_uint16
        L.ref_f32_to_bf16.argtypes = [ctypes.c_uint32]
        L.ref_bf16_to_f32.restype = ctypes.c_uint32
        L.ref_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.ref_f32_to_f16.restype = ctypes.c_uint16
        L.ref_f32_to_f16.argtypes = [ctypes.c_uint32]
        L.ref_f16_to_f32.restype = ctypes.c_uint32
        L.ref_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.ref_flat_copy.restype = None
        L.ref_flat_copy.argtypes = [vp, i32, vp, i32, i64]
        L.ref_flat_div.restype = None
        L.ref_flat_div.argtypes = [vp, i32, i64, dbl]
        L.ref_flat_premul.restype = None
        L.ref_flat_premul.argtypes = [vp, i32, i64, dbl]
        L.ref_post_reduce.restype = None
        L.ref_post_reduce.argtypes = [vp, i32, vp, i32, i64, dbl, i32]
        L.ref_gather_in.restype = None
        L.ref_gather_in.argtypes = [i32, vp, vp, vp, i32, vp, i32, i64, dbl, i32]
        L.ref_scatter_out.restype = None
        L.ref_scatter_out.argtypes = [i32, vp, vp, i32, vp, i32]
        L.ref_adamw_step.restype = None
        L.ref_adamw_step.argtypes = [vp, vp, vp, vp, vp, i32, i64, dbl, dbl, dbl, dbl, dbl, i64, i32, i32,
                                     ctypes.c_float, i32]
        L.ref_sumsq.restype = dbl
        L.ref_sumsq.argtypes = [vp, i32, i64]
        L.ref_clip_coef.restype = None
        L.ref_clip_coef.argtypes = [dbl, dbl, vp]
        L.ref_flat_scale.restype = None
        L.ref_flat_scale.argtypes = [vp, i32, i64, ctypes.c_float]
        _lib = L
    return _lib


def _check(t: torch.Tensor) -> None:
    assert t.device.type == "cpu" and t.is_contiguous()


def flat_copy(dst: torch.Tensor, src: torch.Tensor) -> None:
    _check(dst), _check(src)
    lib().ref_flat_copy(dst.data_ptr(), DT[dst.dtype], src.data_ptr(), DT[src.dtype], dst.numel())


def flat_div(buf: torch.Tensor, factor: float | None) -> None:
    _check(buf)
    if factor is None:
        return
    lib().ref_flat_div(buf.data_ptr(), DT[buf.dtype], buf.numel(), float(factor))


def flat_premul(buf: torch.Tensor, scalar: float) -> None:
    _check(buf)
    lib().ref_flat_premul(buf.data_ptr(), DT[buf.dtype], buf.numel(), float(scalar))


def post_reduce(shard: torch.Tensor, chunk: torch.Tensor, post: float | None, accumulate: bool) -> None:
    _check(shard), _check(chunk)
    lib().ref_post_reduce(
        shard.data_ptr(), DT[shard.dtype], chunk.data_ptr(), DT[chunk.dtype], shard.numel(),
        0.0 if post is None else float(post), int(accumulate),
    )


def _ptr_array(tensors) -> np.ndarray:
    return np.array([t.data_ptr() for t in tensors], dtype=np.uint64)


def gather_in(tensors, modes, offsets, flat: torch.Tensor, t_pad: int, pre: float | None, zero_pad: bool) -> None:
    for t in tensors:
        _check(t)
    _check(flat)
    ptrs = _ptr_array(tensors)
    offs = np.asarray(offsets, dtype=np.int64)
    md = np.asarray(modes, dtype=np.uint8)
    tdt = DT[tensors[0].dtype] if tensors else DT[flat.dtype]
    lib().ref_gather_in(
        len(tensors), ptrs.ctypes.data, offs.ctypes.data, md.ctypes.data, tdt,
        flat.data_ptr(), DT[flat.dtype], int(t_pad), 0.0 if pre is None else float(pre), int(zero_pad),
    )


def scatter_out(tensors, offsets, flat: torch.Tensor) -> None:
    for t in tensors:
        _check(t)
    _check(flat)
    ptrs = _ptr_array(tensors)
    offs = np.asarray(offsets, dtype=np.int64)
    tdt = DT[tensors[0].dtype] if tensors else DT[flat.dtype]
    lib().ref_scatter_out(len(tensors), ptrs.ctypes.data, offs.ctypes.data, tdt, flat.data_ptr(), DT[flat.dtype])


def adamw_step(p, g, m, v, out16, *, lr, beta1, beta2, eps, weight_decay, step, decoupled=True, grad_scale=None,
               zero_grad=False) -> None:
    """One Adam(W) step in place on binary32 CPU tensors; `out16` (bf16/f16 or None) receives round16(p)."""
    for t in (p, g, m, v):
        _check(t)
        assert t.dtype == torch.float32 and t.numel() == p.numel()
    if out16 is not None:
        _check(out16)
    lib().ref_adamw_step(
        p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), None if out16 is None else out16.data_ptr(),
        0 if out16 is None else DT[out16.dtype], p.numel(), float(lr), float(beta1), float(beta2), float(eps),
        float(weight_decay), int(step), int(decoupled), int(grad_scale is not None),
        0.0 if grad_scale is None else float(grad_scale), int(zero_grad),
    )


def sumsq(src: torch.Tensor) -> float:
    _check(src)
    return float(lib().ref_sumsq(src.data_ptr(), DT[src.dtype], src.numel()))


def clip_coef(sumsq_value: float, max_norm: float) -> tuple[float, float]:
    out = np.zeros(2, dtype=np.float32)
    lib().ref_clip_coef(float(sumsq_value), float(max_norm), out.ctypes.data)
    return float(out[0]), float(out[1])


def flat_scale(buf: torch.Tensor, coef: float) -> None:
    _check(buf)
    lib().ref_flat_scale(buf.data_ptr(), DT[buf.dtype], buf.numel(), float(np.float32(coef)))
