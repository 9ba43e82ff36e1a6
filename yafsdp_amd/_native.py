"""ctypes binding of ``libyafsdp_hip.so`` (the C ABI in ``include/yafsdp_hip.h``).

There is no CPU or torch fallback: if the library is missing, importing this
module raises, and every call that fails raises ``RuntimeError`` with the
library's error text.  Tensors enter as raw device pointers and the stream as
the ``hipStream_t`` handle of torch's current stream, so work is enqueued
exactly where the reference's torch ops would have been
(ya_fsdp/_collectives.py:46, 110-111).
"""

from __future__ import annotations

import contextlib
import ctypes
import os
import threading
from typing import Sequence

import numpy as np
import torch  # imported before the library so that both share one HIP runtime

_HERE = os.path.dirname(os.path.abspath(__file__))
# YAFSDP_HIP_LIBRARY points at a library built elsewhere (same C ABI); default: the in-tree build
LIB_PATH = os.environ.get("YAFSDP_HIP_LIBRARY") or os.path.join(_HERE, "libyafsdp_hip.so")

# optional host-side helper (csrc/tensorlist.cpp): validates a tensor list and writes its pointer array in one
# C++ pass; without it the same checks run in Python.  It launches nothing and touches no tensor data.
try:
    from . import _tensorlist
except ImportError:  # not built: the Python checks below do the same work, slower for large tables
    _tensorlist = None

DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
MODE_SKIP, MODE_COPY, MODE_ADD = 0, 1, 2
OPT_FLAT_BLOCKS_PER_CU, OPT_TABLE_BLOCKS_PER_CU, OPT_TABLE_LARGE_LOG2, OPT_SCATTER_TILE = 0, 1, 2, 3
OPT_GATHER_TAIL_MB, OPT_SCATTER_TAIL_MB, OPT_FLAT_TAIL_MB, OPT_POST_REDUCE_TAIL_MB = 4, 5, 6, 7

# every symbol include/yafsdp_hip.h declares
EXPORTED_SYMBOLS = (
    "yafsdp_version",
    "yafsdp_error_string",
    "yafsdp_flat_copy",
    "yafsdp_flat_copy_bytes",
    "yafsdp_flat_div",
    "yafsdp_flat_div_copy",
    "yafsdp_post_reduce",
    "yafsdp_flat_premul",
    "yafsdp_post_reduce_premul",
    "yafsdp_post_reduce_sumsq_count",
    "yafsdp_post_reduce_sumsq",
    "yafsdp_post_reduce_fragments",
    "yafsdp_table_create",
    "yafsdp_table_destroy",
    "yafsdp_table_info",
    "yafsdp_gather_in",
    "yafsdp_scatter_out",
    "yafsdp_copy_in_scatter_out",
    "yafsdp_gather_in_post_reduce",
    "yafsdp_flat_copy_fanout",
    "yafsdp_post_reduce_fanin",
    "yafsdp_post_reduce_fanin_premul",
    "yafsdp_binding_create",
    "yafsdp_binding_destroy",
    "yafsdp_gather_in_bound",
    "yafsdp_scatter_out_bound",
    "yafsdp_flat_fill",
    "yafsdp_sumsq_workspace_bytes",
    "yafsdp_flat_sumsq",
    "yafsdp_flat_sumsq_static_max_numel",
    "yafsdp_flat_sumsq_static",
    "yafsdp_sumsq_partials",
    "yafsdp_sumsq_reduce_partials",
    "yafsdp_clip_coef_from_partials",
    "yafsdp_clip_coef",
    "yafsdp_flat_scale",
    "yafsdp_adamw_step",
    "yafsdp_time_next_launch",
    "yafsdp_complete_next_launch",
    "yafsdp_complete_next_launch_pending",
    "yafsdp_trace_next_flat_launch",
    "yafsdp_set_option",
    "yafsdp_get_option",
    "yafsdp_table_set_option",
    "yafsdp_table_get_option",
)


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m yafsdp_amd._build` "
            "(hipcc, gfx950). There is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    vp, i64, dbl, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_double, ctypes.c_int
    lib.yafsdp_version.restype = i32
    lib.yafsdp_version.argtypes = []
    lib.yafsdp_error_string.restype = ctypes.c_char_p
    lib.yafsdp_error_string.argtypes = [i32]
    lib.yafsdp_flat_copy.restype = i32
    lib.yafsdp_flat_copy.argtypes = [vp, i32, vp, i32, i64, vp]
    lib.yafsdp_flat_copy_bytes.restype = i32
    lib.yafsdp_flat_copy_bytes.argtypes = [vp, vp, i64, vp]
    lib.yafsdp_flat_div.restype = i32
    lib.yafsdp_flat_div.argtypes = [vp, i32, i64, dbl, vp]
    lib.yafsdp_flat_div_copy.restype = i32
    lib.yafsdp_flat_div_copy.argtypes = [vp, i32, vp, i32, i64, dbl, vp]
    lib.yafsdp_post_reduce.restype = i32
    lib.yafsdp_post_reduce.argtypes = [vp, i32, vp, i32, i64, dbl, i32, vp]
    lib.yafsdp_flat_premul.restype = i32
    lib.yafsdp_flat_premul.argtypes = [vp, i32, i64, dbl, vp]
    lib.yafsdp_post_reduce_premul.restype = i32
    lib.yafsdp_post_reduce_premul.argtypes = [vp, i32, vp, i32, i64, dbl, i32, vp]
    lib.yafsdp_post_reduce_sumsq_count.restype = i64
    lib.yafsdp_post_reduce_sumsq_count.argtypes = [i64]
    lib.yafsdp_post_reduce_sumsq.restype = i32
    lib.yafsdp_post_reduce_sumsq.argtypes = [vp, i32, vp, i32, i64, dbl, i32, vp, i64, ctypes.POINTER(i64), vp]
    lib.yafsdp_post_reduce_fragments.restype = i32
    lib.yafsdp_post_reduce_fragments.argtypes = [vp, i32, vp, i32, i32, vp, vp, dbl, vp]
    lib.yafsdp_table_create.restype = i32
    lib.yafsdp_table_create.argtypes = [i32, vp, i64, ctypes.POINTER(vp)]
    lib.yafsdp_table_destroy.restype = i32
    lib.yafsdp_table_destroy.argtypes = [vp]
    lib.yafsdp_table_info.restype = i32
    lib.yafsdp_table_info.argtypes = [vp, ctypes.POINTER(i32), ctypes.POINTER(i64), ctypes.POINTER(i64)]
    lib.yafsdp_gather_in.restype = i32
    lib.yafsdp_gather_in.argtypes = [vp, vp, vp, i32, vp, i32, dbl, i32, vp]
    lib.yafsdp_scatter_out.restype = i32
    lib.yafsdp_scatter_out.argtypes = [vp, vp, i32, vp, vp, i32, vp]
    lib.yafsdp_copy_in_scatter_out.restype = i32
    lib.yafsdp_copy_in_scatter_out.argtypes = [vp, vp, i32, vp, vp, vp, vp, i32, i64, vp]
    lib.yafsdp_gather_in_post_reduce.restype = i32
    lib.yafsdp_gather_in_post_reduce.argtypes = [vp, vp, vp, i32, vp, i32, dbl, dbl, dbl, i32, vp, i32, i32, vp]
    lib.yafsdp_flat_copy_fanout.restype = i32
    lib.yafsdp_flat_copy_fanout.argtypes = [vp, i32, i32, vp, i32, i64, vp]
    lib.yafsdp_post_reduce_fanin.restype = i32
    lib.yafsdp_post_reduce_fanin.argtypes = [vp, i32, vp, i32, i32, i64, dbl, i32, vp]
    lib.yafsdp_post_reduce_fanin_premul.restype = i32
    lib.yafsdp_post_reduce_fanin_premul.argtypes = [vp, i32, vp, i32, i32, i64, dbl, i32, vp]
    lib.yafsdp_binding_create.restype = i32
    lib.yafsdp_binding_create.argtypes = [vp, vp, vp, i32, ctypes.POINTER(vp)]
    lib.yafsdp_binding_destroy.restype = i32
    lib.yafsdp_binding_destroy.argtypes = [vp]
    lib.yafsdp_gather_in_bound.restype = i32
    lib.yafsdp_gather_in_bound.argtypes = [vp, vp, i32, dbl, i32, vp]
    lib.yafsdp_scatter_out_bound.restype = i32
    lib.yafsdp_scatter_out_bound.argtypes = [vp, vp, i32, vp]
    lib.yafsdp_flat_fill.restype = i32
    lib.yafsdp_flat_fill.argtypes = [vp, i32, i64, dbl, vp]
    lib.yafsdp_sumsq_workspace_bytes.restype = ctypes.c_size_t
    lib.yafsdp_sumsq_workspace_bytes.argtypes = []
    lib.yafsdp_flat_sumsq.restype = i32
    lib.yafsdp_flat_sumsq.argtypes = [vp, i32, i64, vp, i32, vp, ctypes.c_size_t, vp]
    lib.yafsdp_flat_sumsq_static_max_numel.restype = i64
    lib.yafsdp_flat_sumsq_static_max_numel.argtypes = []
    lib.yafsdp_flat_sumsq_static.restype = i32
    lib.yafsdp_flat_sumsq_static.argtypes = [vp, i32, i64, vp, i32, vp]
    lib.yafsdp_sumsq_partials.restype = i32
    lib.yafsdp_sumsq_partials.argtypes = [vp, i32, i64, vp, i64, ctypes.POINTER(i64), vp]
    lib.yafsdp_sumsq_reduce_partials.restype = i32
    lib.yafsdp_sumsq_reduce_partials.argtypes = [vp, i64, vp, i64, ctypes.POINTER(i64), vp]
    lib.yafsdp_clip_coef_from_partials.restype = i32
    lib.yafsdp_clip_coef_from_partials.argtypes = [vp, i64, dbl, vp, vp, vp]
    lib.yafsdp_clip_coef.restype = i32
    lib.yafsdp_clip_coef.argtypes = [vp, dbl, vp, vp]
    lib.yafsdp_flat_scale.restype = i32
    lib.yafsdp_flat_scale.argtypes = [vp, i32, i64, vp, vp]
    lib.yafsdp_adamw_step.restype = i32
    lib.yafsdp_adamw_step.argtypes = [vp, vp, vp, vp, vp, i32, i64, dbl, dbl, dbl, dbl, dbl, i64, vp, i32, vp]
    lib.yafsdp_time_next_launch.restype = i32
    lib.yafsdp_time_next_launch.argtypes = [vp, vp]
    lib.yafsdp_complete_next_launch.restype = i32
    lib.yafsdp_complete_next_launch.argtypes = [vp]
    lib.yafsdp_complete_next_launch_pending.restype = i32
    lib.yafsdp_complete_next_launch_pending.argtypes = []
    lib.yafsdp_trace_next_flat_launch.restype = i32
    lib.yafsdp_trace_next_flat_launch.argtypes = [vp, i64, ctypes.POINTER(i64)]
    lib.yafsdp_set_option.restype = i32
    lib.yafsdp_set_option.argtypes = [i32, i32]
    lib.yafsdp_get_option.restype = i32
    lib.yafsdp_get_option.argtypes = [i32, ctypes.POINTER(i32)]
    lib.yafsdp_table_set_option.restype = i32
    lib.yafsdp_table_set_option.argtypes = [vp, i32, i32]
    lib.yafsdp_table_get_option.restype = i32
    lib.yafsdp_table_get_option.argtypes = [vp, i32, ctypes.POINTER(i32)]
    return lib


lib = _load()


def error_string(code: int) -> str:
    return lib.yafsdp_error_string(int(code)).decode()


ERR_BUSY = -7  # YAFSDP_ERR_BUSY: every staging slot of a table is held by a queued call
ERR_UNSUPPORTED = -8  # YAFSDP_ERR_UNSUPPORTED: a fused entry point does not serve this table / dtype combination


def _check(code: int, what: str) -> None:
    if code != 0:
        raise RuntimeError(f"{what} failed: {error_string(code)} (code {code})")


def _dt(t: torch.Tensor) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}: the buffer path handles float32, bfloat16, float16") from None


def _flat_arg(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.device.type != "cuda":
        raise RuntimeError(f"{what} must live on the GPU, got {t.device}: this path has no CPU implementation")
    if not t.is_contiguous():
        raise NotImplementedError(f"{what} must be contiguous: shape={tuple(t.shape)} stride={t.stride()}")
    return t


_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_NO_SWITCH = contextlib.nullcontext()


def _stream(t: torch.Tensor) -> int:
    """``hipStream_t`` of torch's current stream on the tensor's device."""
    if _raw_current_stream is not None:  # the handle itself, without building a Stream object (2 us less per call)
        index = t.device.index
        return _raw_current_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(t.device).cuda_stream


def _on(device: torch.device):
    """Context that makes ``device`` current for a library call; free when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def _factor(f: float | None) -> float:
    return 0.0 if f is None else float(f)


# ------------------------------------------------------------------ flat ops --
def flat_copy(dst: torch.Tensor, src: torch.Tensor) -> None:
    """``dst.copy_(src)`` for contiguous tensors of equal numel.  Two tensors of one dtype outside the arithmetic
    dtypes of the path (float8, int8, uint8, ...) are copied as bytes."""
    _flat_arg(dst, "dst"), _flat_arg(src, "src")
    if dst.numel() != src.numel():
        raise ValueError(f"numel mismatch: {dst.numel()} vs {src.numel()}")
    if dst.dtype == src.dtype and dst.dtype not in DTYPE_CODE:
        if dst.device != src.device:
            raise RuntimeError(f"dst on {dst.device}, src on {src.device}")
        with _on(dst.device):
            _check(
                lib.yafsdp_flat_copy_bytes(dst.data_ptr(), src.data_ptr(), dst.numel() * dst.element_size(), _stream(dst)),
                "yafsdp_flat_copy_bytes",
            )
        return
    with _on(dst.device):
        _check(
            lib.yafsdp_flat_copy(dst.data_ptr(), _dt(dst), src.data_ptr(), _dt(src), dst.numel(), _stream(dst)),
            "yafsdp_flat_copy",
        )


def flat_div(buf: torch.Tensor, factor: float | None) -> None:
    """``_div_if_needed(buf, factor)``."""
    _flat_arg(buf, "buf")
    with _on(buf.device):
        _check(
            lib.yafsdp_flat_div(buf.data_ptr(), _dt(buf), buf.numel(), _factor(factor), _stream(buf)),
            "yafsdp_flat_div",
        )


def flat_div_copy(dst: torch.Tensor, src: torch.Tensor, divisor: float) -> None:
    """``dst.copy_(src / divisor)`` for any finite non-zero divisor."""
    _flat_arg(dst, "dst"), _flat_arg(src, "src")
    if dst.numel() != src.numel():
        raise ValueError(f"numel mismatch: {dst.numel()} vs {src.numel()}")
    with _on(dst.device):
        _check(
            lib.yafsdp_flat_div_copy(
                dst.data_ptr(), _dt(dst), src.data_ptr(), _dt(src), dst.numel(), float(divisor), _stream(dst)
            ),
            "yafsdp_flat_div_copy",
        )


def post_reduce(shard: torch.Tensor, chunk: torch.Tensor, post_factor: float | None, accumulate: bool) -> None:
    _flat_arg(shard, "shard"), _flat_arg(chunk, "chunk")
    if shard.numel() != chunk.numel():
        raise ValueError(f"numel mismatch: {shard.numel()} vs {chunk.numel()}")
    with _on(shard.device):
        _check(
            lib.yafsdp_post_reduce(
                shard.data_ptr(), _dt(shard), chunk.data_ptr(), _dt(chunk), shard.numel(),
                _factor(post_factor), int(bool(accumulate)), _stream(shard),
            ),
            "yafsdp_post_reduce",
        )


def flat_premul(buf: torch.Tensor, scalar: float) -> None:
    """``buf *= dtype(scalar)`` in place, rounded to the dtype: one rank's share of a pre-multiplied sum (what the
    collective's AVG / ``_make_nccl_premul_sum`` reduction does to every contribution before adding them up)."""
    _flat_arg(buf, "buf")
    with _on(buf.device):
        _check(
            lib.yafsdp_flat_premul(buf.data_ptr(), _dt(buf), buf.numel(), float(scalar), _stream(buf)),
            "yafsdp_flat_premul",
        )


def post_reduce_premul(shard: torch.Tensor, chunk: torch.Tensor, scalar: float, accumulate: bool) -> None:
    """``post_reduce`` whose chunk first takes the collective's pre-multiplication (``flat_premul``) instead of a
    post-divide; the chunk itself is not written."""
    _flat_arg(shard, "shard"), _flat_arg(chunk, "chunk")
    if shard.numel() != chunk.numel():
        raise ValueError(f"numel mismatch: {shard.numel()} vs {chunk.numel()}")
    with _on(shard.device):
        _check(
            lib.yafsdp_post_reduce_premul(
                shard.data_ptr(), _dt(shard), chunk.data_ptr(), _dt(chunk), shard.numel(),
                float(scalar), int(bool(accumulate)), _stream(shard),
            ),
            "yafsdp_post_reduce_premul",
        )


def post_reduce_sumsq_count(numel: int) -> int:
    """Partial sums ``post_reduce_sumsq`` writes at most for a shard of ``numel`` elements."""
    return int(lib.yafsdp_post_reduce_sumsq_count(int(numel)))


def post_reduce_sumsq(
    shard: torch.Tensor, chunk: torch.Tensor, post_factor: float | None, accumulate: bool, partials: torch.Tensor,
    offset: int = 0,
) -> int:
    """``post_reduce`` that also writes the per-workgroup sums of squares of the resulting shard into
    ``partials[offset:]`` (float64); returns the new offset."""
    _flat_arg(shard, "shard"), _flat_arg(chunk, "chunk"), _flat_arg(partials, "partials")
    if shard.numel() != chunk.numel():
        raise ValueError(f"numel mismatch: {shard.numel()} vs {chunk.numel()}")
    if partials.dtype != torch.float64 or partials.device != shard.device:
        raise TypeError("partials must be a float64 tensor on the shard's device")
    capacity = partials.numel() - offset
    written = ctypes.c_int64()
    with _on(shard.device):
        _check(
            lib.yafsdp_post_reduce_sumsq(
                shard.data_ptr(), _dt(shard), chunk.data_ptr(), _dt(chunk), shard.numel(), _factor(post_factor),
                int(bool(accumulate)), partials.data_ptr() + 8 * offset, max(capacity, 0), ctypes.byref(written),
                _stream(shard),
            ),
            "yafsdp_post_reduce_sumsq",
        )
    return offset + written.value


def post_reduce_fragments(
    shard: torch.Tensor, chunk: torch.Tensor, frag_numels: Sequence[int], frag_modes: Sequence[int],
    post_factor: float | None,
) -> None:
    _flat_arg(shard, "shard"), _flat_arg(chunk, "chunk")
    numels = np.ascontiguousarray(frag_numels, dtype=np.int64)
    modes = np.ascontiguousarray(frag_modes, dtype=np.uint8)
    if numels.shape != modes.shape:
        raise ValueError("frag_numels and frag_modes differ in length")
    if int(numels.sum()) > min(shard.numel(), chunk.numel()):
        raise ValueError("fragments exceed the shard")
    with _on(shard.device):
        _check(
            lib.yafsdp_post_reduce_fragments(
                shard.data_ptr(), _dt(shard), chunk.data_ptr(), _dt(chunk), int(numels.size),
                numels.ctypes.data, modes.ctypes.data, _factor(post_factor), _stream(shard),
            ),
            "yafsdp_post_reduce_fragments",
        )


# --------------------------------------------------------------- table ops --
def all_contiguous(tensors: Sequence[torch.Tensor | None]) -> bool:
    """True if every tensor of the list (``None`` entries aside) is contiguous."""
    if _tensorlist is not None and isinstance(tensors, (list, tuple)):
        return _tensorlist.all_contiguous(tensors)
    return all(t is None or t.is_contiguous() for t in tensors)


class TensorTable:
    """Device-resident metadata of one flat buffer (tensor boundaries and the
    tile -> tensor map).  Static for the life of a parameter group; the tensor
    pointers are passed with every call.  Tables with more than 16 tensors pass
    them through 8 staging slots; a call with the same tensors as an earlier
    one reuses its slot.  Only when 8 calls with 8 different tensor sets are
    still queued does a further call wait (for the current stream) before it
    stages its own."""

    def __init__(self, numels: Sequence[int], padded_numel: int, device: torch.device):
        self.numels = [int(n) for n in numels]
        self.total_numel = sum(self.numels)
        self.padded_numel = int(padded_numel)
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError(f"TensorTable needs a GPU device, got {device}")
        if self.device.index is None:  # "cuda" means the current GPU; tensors always report an indexed device
            self.device = torch.device("cuda", torch.cuda.current_device())
        arr = np.ascontiguousarray(self.numels, dtype=np.int64)
        handle = ctypes.c_void_p()
        with _on(self.device):
            _check(
                lib.yafsdp_table_create(len(self.numels), arr.ctypes.data, self.padded_numel, ctypes.byref(handle)),
                "yafsdp_table_create",
            )
        self._handle = handle
        self._init_host_arrays()

    def _init_host_arrays(self) -> None:
        """Per-call pointer / mode arrays (``numels`` and ``device`` are set); the lock keeps "fill, then launch"
        atomic when the table is used from two host threads (the main thread and the autograd engine thread)."""
        self._numels_arr = np.ascontiguousarray(self.numels, dtype=np.int64)
        self._ptrs = np.zeros(max(1, len(self.numels)), dtype=np.uint64)
        self._modes = np.zeros(max(1, len(self.numels)), dtype=np.uint8)
        # their addresses, looked up once (numpy's .ctypes builds an object per access: 0.4 us each, five per call)
        self._numels_addr = self._numels_arr.ctypes.data
        self._ptrs_addr = self._ptrs.ctypes.data
        self._modes_addr = self._modes.ctypes.data
        self._on_cuda = self.device.type == "cuda"
        self._device_index = self.device.index if self.device.index is not None else -1
        self._lock = threading.Lock()

    def close(self) -> None:
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            lib.yafsdp_table_destroy(h)

    def set_option(self, option: int, value: int) -> None:
        """This table's own write-through tail (``OPT_GATHER_TAIL_MB`` / ``OPT_SCATTER_TAIL_MB``) in megabytes; it
        takes precedence over the process-wide option in every call on this table.  -1: follow the process-wide
        option again."""
        _check(lib.yafsdp_table_set_option(self._handle, int(option), int(value)), "yafsdp_table_set_option")

    def get_option(self, option: int) -> int:
        v = ctypes.c_int()
        _check(lib.yafsdp_table_get_option(self._handle, int(option), ctypes.byref(v)), "yafsdp_table_get_option")
        return v.value

    def bind(self, tensors: Sequence[torch.Tensor | None], modes: Sequence[int] | None = None) -> "TensorBinding":
        """Fix the tensor side for many calls (see ``TensorBinding``)."""
        return TensorBinding(self, tensors, modes)

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass

    def _fill(self, tensors: Sequence[torch.Tensor | None], modes: Sequence[int] | None, what: str) -> int:
        """Write the per-call pointer and mode arrays; returns the dtype code of
        the tensors (-1 if every tensor is skipped).  Checks run as whole-list
        passes (one Python-level loop each) so that a table with thousands of
        tensors costs a fraction of a millisecond, not several."""
        n = len(self.numels)
        if len(tensors) != n:
            raise ValueError(f"{what}: expected {n} tensors, got {len(tensors)}")
        if modes is not None and len(modes) != n:
            raise ValueError(f"{what}: expected {n} modes, got {len(modes)}")
        if n == 0:
            return -1
        if _tensorlist is not None:
            code = _tensorlist.fill(
                tensors, modes, self._numels_addr, self._ptrs_addr, self._modes_addr, self._on_cuda, self._device_index,
            )
            if code != _tensorlist.REJECTED:
                return code
            # not accepted as it stands: the checks below find out why and raise
        if modes is None:
            live = [t for t in tensors if t is not None]
            if len(live) == n:
                self._modes[:n] = MODE_COPY
            else:
                self._modes[:n] = [MODE_SKIP if t is None else MODE_COPY for t in tensors]
        else:
            self._modes[:n] = [MODE_SKIP if t is None else int(m) for t, m in zip(tensors, modes)]
            live = [t for t, m in zip(tensors, self._modes[:n].tolist()) if m != MODE_SKIP]
        if not live:
            self._ptrs[:n] = 0
            return -1
        dtypes = {t.dtype for t in live}
        if len(dtypes) != 1:
            raise TypeError(f"{what}: tensors of one call share a dtype, got {sorted(map(str, dtypes))}")
        dtype = next(iter(dtypes))
        if dtype not in DTYPE_CODE:
            _dt(live[0])
        if len(live) == n:
            numels = [t.numel() for t in live]
            if numels != self.numels:
                p = next(i for i, (a, b) in enumerate(zip(numels, self.numels)) if a != b)
                raise ValueError(f"{what}[{p}]: numel {numels[p]} != {self.numels[p]}")
            self._ptrs[:n] = [t.data_ptr() for t in live]
        else:
            for p, t in enumerate(tensors):
                if self._modes[p] == MODE_SKIP:
                    self._ptrs[p] = 0
                    continue
                if t.numel() != self.numels[p]:
                    raise ValueError(f"{what}[{p}]: numel {t.numel()} != {self.numels[p]}")
                self._ptrs[p] = t.data_ptr()
        if not all(t.is_contiguous() for t in live):
            p = next(i for i, t in enumerate(tensors) if t is not None and not t.is_contiguous())
            _flat_arg(tensors[p], f"{what}[{p}]")
        devices = {t.device for t in live}
        if devices != {self.device}:
            bad = next(d for d in devices if d != self.device)
            if bad.type != "cuda":
                raise RuntimeError(f"{what} must live on the GPU, got {bad}: this path has no CPU implementation")
            raise RuntimeError(f"{what} holds a tensor on {bad}, table on {self.device}")
        return DTYPE_CODE[dtype]

    def gather_in(
        self, tensors: Sequence[torch.Tensor | None], flat: torch.Tensor, modes: Sequence[int] | None = None,
        pre_factor: float | None = None, zero_pad: bool = True,
    ) -> None:
        """Reduce copy-in (+ fused pre-divide and pad zero-fill) into ``flat``."""
        _flat_arg(flat, "flat")
        if flat.numel() < self.padded_numel:
            raise ValueError(f"flat buffer holds {flat.numel()} elements, table needs {self.padded_numel}")
        with self._lock, _on(self.device):
            tdt = self._fill(tensors, modes, "tensors")
            if tdt < 0:
                tdt = _dt(flat)
            args = (self._handle, self._ptrs_addr, self._modes_addr, tdt, flat.data_ptr(), _dt(flat),
                    _factor(pre_factor), int(bool(zero_pad)), _stream(flat))
            code = lib.yafsdp_gather_in(*args)
            if code == ERR_BUSY:  # back-pressure: 8 calls with different tensor sets are still queued on this table
                torch.cuda.current_stream(self.device).synchronize()
                code = lib.yafsdp_gather_in(*args)
            _check(code, "yafsdp_gather_in")

    def copy_in_scatter_out(
        self, flat: torch.Tensor, tensors: Sequence[torch.Tensor | None], ag_in: torch.Tensor, master: torch.Tensor,
        modes: Sequence[int] | None = None,
    ) -> bool:
        """``flat_copy(ag_in, master)`` and ``scatter_out(flat, tensors)`` as ONE launch (two independent jobs in
        one grid).  Returns False without launching anything when the tensors' dtype differs from the gathered
        buffer's (``scatter_out`` casts; this launch does not); the caller then makes the two calls."""
        _flat_arg(flat, "flat"), _flat_arg(ag_in, "ag_in"), _flat_arg(master, "master")
        if flat.numel() < self.total_numel:
            raise ValueError(f"flat buffer holds {flat.numel()} elements, table needs {self.total_numel}")
        if ag_in.numel() != master.numel() or ag_in.dtype != flat.dtype:
            raise ValueError("ag_in must have the master shard's element count and the gathered buffer's dtype")
        with self._lock, _on(self.device):
            tdt = self._fill(tensors, modes, "tensors")
            if tdt >= 0 and tdt != _dt(flat):
                return False
            args = (self._handle, flat.data_ptr(), _dt(flat), self._ptrs_addr, self._modes_addr,
                    ag_in.data_ptr(), master.data_ptr(), _dt(master), master.numel(), _stream(flat))
            code = lib.yafsdp_copy_in_scatter_out(*args)
            if code == ERR_BUSY:  # back-pressure, as in gather_in
                torch.cuda.current_stream(self.device).synchronize()
                code = lib.yafsdp_copy_in_scatter_out(*args)
        if code == ERR_UNSUPPORTED:
            return False
        _check(code, "yafsdp_copy_in_scatter_out")
        return True

    def gather_in_post_reduce(
        self, tensors: Sequence[torch.Tensor | None], flat: torch.Tensor, shard: torch.Tensor, accumulate: bool,
        modes: Sequence[int] | None = None, zero_pad: bool = True, pre_factor: float | None = None,
        post_factor: float | None = None, custom_divisor: float | None = None,
    ) -> bool:
        """Reduce copy-in into ``flat`` and post-reduce of the whole buffer into ``shard`` as ONE launch: what a
        shard group of size one does between backward and optimizer (no collective in between).  ``pre_factor`` and
        ``post_factor`` follow ``_div_if_needed`` (applied if > 1); ``custom_divisor`` is the division by a custom
        gradient divide factor of such a group (any value; excludes the other two).  Returns False without launching
        anything when the library does not serve the dtype combination (a reduce buffer that has neither the
        gradients' dtype nor float32)."""
        _flat_arg(flat, "flat"), _flat_arg(shard, "shard")
        if flat.numel() < self.padded_numel or shard.numel() != self.padded_numel:
            raise ValueError(f"flat / shard hold {flat.numel()} / {shard.numel()} elements, table needs {self.padded_numel}")
        with self._lock, _on(self.device):
            tdt = self._fill(tensors, modes, "tensors")
            if tdt < 0:
                tdt = _dt(flat)
            args = (self._handle, self._ptrs_addr, self._modes_addr, tdt, flat.data_ptr(), _dt(flat),
                    _factor(pre_factor), _factor(custom_divisor), _factor(post_factor),
                    int(bool(zero_pad)), shard.data_ptr(), _dt(shard), int(bool(accumulate)), _stream(flat))
            code = lib.yafsdp_gather_in_post_reduce(*args)
            if code == ERR_BUSY:  # back-pressure, as in gather_in
                torch.cuda.current_stream(self.device).synchronize()
                code = lib.yafsdp_gather_in_post_reduce(*args)
        if code == ERR_UNSUPPORTED:
            return False
        _check(code, "yafsdp_gather_in_post_reduce")
        return True

    def scatter_out(
        self, flat: torch.Tensor, tensors: Sequence[torch.Tensor | None], modes: Sequence[int] | None = None
    ) -> None:
        """Materialising copy-out of ``flat[:total]`` into ``tensors``."""
        _flat_arg(flat, "flat")
        if flat.numel() < self.total_numel:
            raise ValueError(f"flat buffer holds {flat.numel()} elements, table needs {self.total_numel}")
        with self._lock, _on(self.device):
            tdt = self._fill(tensors, modes, "tensors")
            if tdt < 0:
                return
            args = (self._handle, flat.data_ptr(), _dt(flat), self._ptrs_addr, self._modes_addr, tdt,
                    _stream(flat))
            code = lib.yafsdp_scatter_out(*args)
            if code == ERR_BUSY:  # back-pressure, as in gather_in
                torch.cuda.current_stream(self.device).synchronize()
                code = lib.yafsdp_scatter_out(*args)
            _check(code, "yafsdp_scatter_out")


def flat_copy_fanout(dsts: Sequence[torch.Tensor], src: torch.Tensor) -> None:
    """``d.copy_(src)`` for every ``d`` in ``dsts`` in one pass over ``src`` (at most 16 destinations)."""
    _flat_arg(src, "src")
    if not dsts:
        raise ValueError("at least one destination")
    for d in dsts:
        _flat_arg(d, "dst")
        if d.numel() != src.numel() or d.dtype != dsts[0].dtype or d.device != src.device:
            raise ValueError("destinations must match the source's size and device and share a dtype")
    ptrs = (ctypes.c_void_p * len(dsts))(*[d.data_ptr() for d in dsts])
    with _on(src.device):
        _check(
            lib.yafsdp_flat_copy_fanout(ptrs, len(dsts), _dt(dsts[0]), src.data_ptr(), _dt(src), src.numel(), _stream(src)),
            "yafsdp_flat_copy_fanout",
        )


def post_reduce_fanin(
    shard: torch.Tensor, chunks: Sequence[torch.Tensor], post_factor: float | None, accumulate: bool,
    *, premul: float | None = None,
) -> None:
    """``shard (+)= div(round(sum of chunks in float32))``: the reduce-scatter of the ranks' chunks, the
    post-divide and the accumulation into the gradient shard in one pass (at most 16 chunks).  ``premul``: the
    scalar of a collective that scales inside the reduction (``ReduceOp.AVG``: 1 / ranks) - every chunk element is
    multiplied by it, rounded to the chunk dtype, before the sum; there is no post-divide then."""
    _flat_arg(shard, "shard")
    if not chunks:
        raise ValueError("at least one chunk")
    if premul is not None and post_factor is not None:
        raise ValueError("a collective that scales inside the reduction has no post-divide")
    for c in chunks:
        _flat_arg(c, "chunk")
        if c.numel() != shard.numel() or c.dtype != chunks[0].dtype or c.device != shard.device:
            raise ValueError("chunks must match the shard's size and device and share a dtype")
    ptrs = (ctypes.c_void_p * len(chunks))(*[c.data_ptr() for c in chunks])
    head = (shard.data_ptr(), _dt(shard), ptrs, len(chunks), _dt(chunks[0]), shard.numel())
    with _on(shard.device):
        if premul is not None:
            _check(
                lib.yafsdp_post_reduce_fanin_premul(*head, float(premul), int(bool(accumulate)), _stream(shard)),
                "yafsdp_post_reduce_fanin_premul",
            )
        else:
            _check(
                lib.yafsdp_post_reduce_fanin(*head, _factor(post_factor), int(bool(accumulate)), _stream(shard)),
                "yafsdp_post_reduce_fanin",
            )


class TensorBinding:
    """The tensor side of a ``TensorTable`` fixed for many calls (tensors that
    persist across steps: copy-out destinations, gradient accumulators).
    Pointers, modes and dtype are checked and staged once; ``gather_in`` /
    ``scatter_out`` then cost one launch and no per-tensor host work, and can be
    captured into a HIP graph whatever the table size.  Holds references to the
    tensors and the table."""

    def __init__(self, table: "TensorTable", tensors: Sequence[torch.Tensor | None], modes: Sequence[int] | None = None):
        self.table = table
        self.tensors = list(tensors)
        handle = ctypes.c_void_p()
        with table._lock, _on(table.device):
            tdt = table._fill(self.tensors, modes, "tensors")
            self._all_skipped = tdt < 0
            _check(
                lib.yafsdp_binding_create(
                    table._handle, table._ptrs_addr, table._modes_addr, max(tdt, 0), ctypes.byref(handle)
                ),
                "yafsdp_binding_create",
            )
        self._handle = handle

    def close(self) -> None:
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            lib.yafsdp_binding_destroy(h)

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass

    def gather_in(self, flat: torch.Tensor, pre_factor: float | None = None, zero_pad: bool = True) -> None:
        _flat_arg(flat, "flat")
        if flat.numel() < self.table.padded_numel:
            raise ValueError(f"flat buffer holds {flat.numel()} elements, table needs {self.table.padded_numel}")
        with _on(self.table.device):
            _check(
                lib.yafsdp_gather_in_bound(
                    self._handle, flat.data_ptr(), _dt(flat), _factor(pre_factor), int(bool(zero_pad)), _stream(flat)
                ),
                "yafsdp_gather_in_bound",
            )

    def scatter_out(self, flat: torch.Tensor) -> None:
        _flat_arg(flat, "flat")
        if flat.numel() < self.table.total_numel:
            raise ValueError(f"flat buffer holds {flat.numel()} elements, table needs {self.table.total_numel}")
        if self._all_skipped:
            return
        with _on(self.table.device):
            _check(
                lib.yafsdp_scatter_out_bound(self._handle, flat.data_ptr(), _dt(flat), _stream(flat)),
                "yafsdp_scatter_out_bound",
            )


# ---- optimizer-side passes over a flat shard ---------------------------------
ADAM_DECOUPLED_DECAY, ADAM_ZERO_GRAD = 1, 2


def flat_fill(dst: torch.Tensor, value: float = 0.0) -> None:
    """``dst.fill_(value)`` (``zero_()`` by default) on a flat buffer."""
    _flat_arg(dst, "dst")
    with _on(dst.device):
        _check(lib.yafsdp_flat_fill(dst.data_ptr(), _dt(dst), dst.numel(), float(value), _stream(dst)), "yafsdp_flat_fill")


def sumsq_workspace(device: torch.device) -> torch.Tensor:
    """Scratch buffer that ``flat_sumsq`` needs; reusable across calls that do not overlap."""
    return torch.empty(lib.yafsdp_sumsq_workspace_bytes(), dtype=torch.uint8, device=device)


def flat_sumsq(src: torch.Tensor, out: torch.Tensor, workspace: torch.Tensor, accumulate: bool = False) -> None:
    """``out[0] (+)= sum(float(src)**2)`` in binary64; ``out`` is a float64 device tensor."""
    _flat_arg(src, "src"), _flat_arg(out, "out"), _flat_arg(workspace, "workspace")
    if out.dtype != torch.float64 or out.numel() < 1:
        raise TypeError("out must be a float64 tensor with at least one element")
    if out.device != src.device or workspace.device != src.device:
        raise RuntimeError("src, out and workspace must live on one device")
    with _on(src.device):
        _check(
            lib.yafsdp_flat_sumsq(
                src.data_ptr(), _dt(src), src.numel(), out.data_ptr(), int(accumulate), workspace.data_ptr(),
                workspace.numel() * workspace.element_size(), _stream(src),
            ),
            "yafsdp_flat_sumsq",
        )


def flat_sumsq_static(src: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """``flat_sumsq`` without a workspace and without any allocation: the partial sums live in a fixed array inside
    the library (one per GPU), so calls on one GPU must not overlap in time."""
    _flat_arg(src, "src"), _flat_arg(out, "out")
    if out.dtype != torch.float64 or out.numel() < 1:
        raise TypeError("out must be a float64 tensor with at least one element")
    if out.device != src.device:
        raise RuntimeError("src and out must live on one device")
    with _on(src.device):
        _check(
            lib.yafsdp_flat_sumsq_static(src.data_ptr(), _dt(src), src.numel(), out.data_ptr(), int(accumulate), _stream(src)),
            "yafsdp_flat_sumsq_static",
        )


SUMSQ_MAX_PARTIALS = lib.yafsdp_sumsq_workspace_bytes() // 8


def sumsq_partials(src: torch.Tensor, partials: torch.Tensor, offset: int) -> int:
    """Per-workgroup sums of squares of ``src`` into ``partials[offset:]`` (float64); returns the new offset."""
    _flat_arg(src, "src"), _flat_arg(partials, "partials")
    if partials.dtype != torch.float64 or partials.device != src.device:
        raise TypeError("partials must be a float64 tensor on the source's device")
    capacity = partials.numel() - offset
    if capacity < 1:
        raise ValueError("partials is full")
    written = ctypes.c_int64()
    with _on(src.device):
        _check(
            lib.yafsdp_sumsq_partials(
                src.data_ptr(), _dt(src), src.numel(), partials.data_ptr() + 8 * offset, capacity, ctypes.byref(written),
                _stream(src),
            ),
            "yafsdp_sumsq_partials",
        )
    return offset + written.value


def sumsq_reduce_partials(partials: torch.Tensor, count: int, out: torch.Tensor) -> int:
    """``out[b] = sum(partials[4096 b : 4096 (b + 1)])`` over the first ``count`` partial sums; returns how many
    sums ``out`` now holds."""
    _flat_arg(partials, "partials"), _flat_arg(out, "out")
    if partials.dtype != torch.float64 or out.dtype != torch.float64:
        raise TypeError("partial sums are float64")
    if count > partials.numel():
        raise ValueError("count exceeds the partials buffer")
    written = ctypes.c_int64()
    with _on(partials.device):
        _check(
            lib.yafsdp_sumsq_reduce_partials(
                partials.data_ptr(), int(count), out.data_ptr(), out.numel(), ctypes.byref(written), _stream(partials)
            ),
            "yafsdp_sumsq_reduce_partials",
        )
    return written.value


def clip_coef_from_partials(
    partials: torch.Tensor, count: int, max_norm: float, norm_and_coef: torch.Tensor, sumsq: torch.Tensor | None = None
) -> None:
    """Adds ``partials[:count]`` and writes ``{norm, clip coefficient}`` (float32), optionally the sum (float64)."""
    _flat_arg(partials, "partials"), _flat_arg(norm_and_coef, "norm_and_coef")
    if partials.dtype != torch.float64 or norm_and_coef.dtype != torch.float32 or norm_and_coef.numel() < 2:
        raise TypeError("partials must be float64 and norm_and_coef float32 with two elements")
    if not 0 <= count <= partials.numel():
        raise ValueError("count out of range")
    with _on(partials.device):
        _check(
            lib.yafsdp_clip_coef_from_partials(
                partials.data_ptr(), count, float(max_norm), None if sumsq is None else sumsq.data_ptr(),
                norm_and_coef.data_ptr(), _stream(partials),
            ),
            "yafsdp_clip_coef_from_partials",
        )


def clip_coef(sumsq: torch.Tensor, max_norm: float, norm_and_coef: torch.Tensor) -> None:
    """``norm_and_coef[0] = sqrt(sumsq[0])``, ``norm_and_coef[1] = min(max_norm / (norm + 1e-6), 1)`` (float32)."""
    _flat_arg(sumsq, "sumsq"), _flat_arg(norm_and_coef, "norm_and_coef")
    if sumsq.dtype != torch.float64 or norm_and_coef.dtype != torch.float32 or norm_and_coef.numel() < 2:
        raise TypeError("sumsq must be float64 and norm_and_coef float32 with two elements")
    with _on(sumsq.device):
        _check(
            lib.yafsdp_clip_coef(sumsq.data_ptr(), float(max_norm), norm_and_coef.data_ptr(), _stream(sumsq)),
            "yafsdp_clip_coef",
        )


def flat_scale(buf: torch.Tensor, coef: torch.Tensor) -> None:
    """``buf.mul_(coef)`` with a one-element float32 device tensor; a coefficient of exactly 1 costs no traffic."""
    _flat_arg(buf, "buf"), _flat_arg(coef, "coef")
    if coef.dtype != torch.float32 or coef.numel() != 1 or coef.device != buf.device:
        raise TypeError("coef must be a one-element float32 tensor on the buffer's device")
    with _on(buf.device):
        _check(lib.yafsdp_flat_scale(buf.data_ptr(), _dt(buf), buf.numel(), coef.data_ptr(), _stream(buf)), "yafsdp_flat_scale")


def adamw_step(
    param: torch.Tensor,
    grad: torch.Tensor,
    exp_avg: torch.Tensor,
    exp_avg_sq: torch.Tensor,
    out16: torch.Tensor | None,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    eps: float,
    weight_decay: float,
    step: int,
    decoupled: bool = True,
    grad_scale: torch.Tensor | None = None,
    zero_grad: bool = False,
) -> None:
    """One Adam(W) step on a flat float32 shard, fused with the 16-bit copy-in of the next iteration."""
    n = param.numel()
    for name, t in (("param", param), ("grad", grad), ("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
        _flat_arg(t, name)
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be float32, got {t.dtype}")
        if t.numel() != n or t.device != param.device:
            raise ValueError(f"{name}: expected {n} elements on {param.device}")
    out_ptr, out_dt = None, 0
    if out16 is not None:
        _flat_arg(out16, "out16")
        if out16.dtype not in (torch.bfloat16, torch.float16) or out16.numel() != n or out16.device != param.device:
            raise TypeError("out16 must be a bfloat16 / float16 tensor of the shard's size on its device")
        out_ptr, out_dt = out16.data_ptr(), _dt(out16)
    gs_ptr = None
    if grad_scale is not None:
        _flat_arg(grad_scale, "grad_scale")
        if grad_scale.dtype != torch.float32 or grad_scale.numel() != 1 or grad_scale.device != param.device:
            raise TypeError("grad_scale must be a one-element float32 tensor on the shard's device")
        gs_ptr = grad_scale.data_ptr()
    flags = (ADAM_DECOUPLED_DECAY if decoupled else 0) | (ADAM_ZERO_GRAD if zero_grad else 0)
    with _on(param.device):
        _check(
            lib.yafsdp_adamw_step(
                param.data_ptr(), grad.data_ptr(), exp_avg.data_ptr(), exp_avg_sq.data_ptr(), out_ptr, out_dt, n,
                float(lr), float(beta1), float(beta2), float(eps), float(weight_decay), int(step), gs_ptr, flags,
                _stream(param),
            ),
            "yafsdp_adamw_step",
        )


def time_next_launch(start: torch.cuda.Event | None, stop: torch.cuda.Event | None) -> None:
    """Measurement hook: the next kernel launched through the library from this thread carries ``start`` /
    ``stop`` on its own dispatch (kernel begin and end, no launch gap); ``start.elapsed_time(stop)`` after a
    synchronisation is the kernel's duration.  Both events need ``enable_timing=True``."""
    if start is None or stop is None:
        _check(lib.yafsdp_time_next_launch(None, None), "yafsdp_time_next_launch")
        return
    for ev in (start, stop):
        if not ev.cuda_event:  # torch creates the HIP event lazily, on its first record
            ev.record()
    _check(lib.yafsdp_time_next_launch(start.cuda_event, stop.cuda_event), "yafsdp_time_next_launch")


def launch_recording(event: torch.cuda.Event, launch, stream: "torch.cuda.Stream | None" = None) -> torch.cuda.Event:
    """Runs ``launch()`` (ONE call into the library that launches one kernel on the current stream) so that the
    kernel itself records ``event`` at its completion: what ``launch(); event.record()`` does, without the marker
    packet that a recorded event puts behind the kernel in its queue (6.5 us of idle GPU between two kernels of one
    stream, 11 us on a hop to another stream).  A call that turns out to launch nothing records the event the
    ordinary way."""
    stream = stream if stream is not None else torch.cuda.current_stream()
    if torch.cuda.is_current_stream_capturing():  # a captured graph orders its nodes by itself
        launch()
        event.record(stream)
        return event
    if not event.cuda_event:  # torch creates the HIP event lazily, on its first record
        event.record(stream)
    lib.yafsdp_complete_next_launch(event.cuda_event)
    try:
        launch()
    finally:
        if lib.yafsdp_complete_next_launch_pending():
            lib.yafsdp_complete_next_launch(None)
            event.record(stream)
    return event


class FlatLaunchTrace:
    """Per-workgroup timeline of one flat-kernel launch: ``with FlatLaunchTrace(capacity, device) as tr: <one flat
    call>``; afterwards (and after a synchronize) ``tr.times()`` is an ``(n_workgroups, 2)`` int64 tensor of start /
    end counts of the GPU's 100 MHz wall clock."""

    def __init__(self, capacity: int, device: torch.device):
        self.buf = torch.zeros(2 * capacity, dtype=torch.int64, device=device)
        self.capacity = int(capacity)
        self._n = ctypes.c_int64(0)

    def __enter__(self) -> "FlatLaunchTrace":
        _check(lib.yafsdp_trace_next_flat_launch(self.buf.data_ptr(), self.capacity, ctypes.byref(self._n)),
               "yafsdp_trace_next_flat_launch")
        return self

    def __exit__(self, *exc) -> None:
        lib.yafsdp_trace_next_flat_launch(None, 0, None)

    def times(self) -> torch.Tensor:
        if self._n.value <= 0:
            raise RuntimeError(f"no flat launch was traced (grid {-self._n.value} against capacity {self.capacity})")
        return self.buf[: 2 * self._n.value].view(-1, 2).cpu()


def set_option(option: int, value: int) -> None:
    _check(lib.yafsdp_set_option(int(option), int(value)), "yafsdp_set_option")


def get_option(option: int) -> int:
    v = ctypes.c_int()
    _check(lib.yafsdp_get_option(int(option), ctypes.byref(v)), "yafsdp_get_option")
    return v.value


# Store policies: how many megabytes at the END of each kind of kernel's output are stored write-through (the rest
# non-temporal), as (flat copies / casts / divides, post-reduce, scatter-out, gather-in).  Written-through lines
# stay in the 256-MB memory-side cache until later traffic evicts them; they pay if they are still there when their
# buffer is touched again (a read is served from the cache, a write overwrites them before they reached DRAM) and
# cost if they are evicted in the middle of other kernels:
#   "rotating_sets"  the library's own defaults, cache-neutral: parameter groups taking turns on shared buffers
#                    (ya_fsdp/_state.py:636-652), up to four reduce buffers in rotation.  Only the reduce copy-in
#                    writes its last 64 MB through (the gradient buffers come round soonest); `fully_shard` sizes
#                    that tail per group from the number of gradient buffers of its model (``TensorTable.set_option``).
#   "single_set"     opt-in: one set of buffers rewritten step after step (a loop over one layer).  The flat kernels
#                    write through everywhere and the reduce copy-in its last 96 MB, and the loop finds its own
#                    output in that cache, which a training run over many groups does not.
_EVERYTHING = 1 << 20
STORE_POLICIES = {"rotating_sets": (0, 0, 0, 64), "single_set": (_EVERYTHING, _EVERYTHING, 0, 96)}
_STORE_POLICY_OPTIONS = (OPT_FLAT_TAIL_MB, OPT_POST_REDUCE_TAIL_MB, OPT_SCATTER_TAIL_MB, OPT_GATHER_TAIL_MB)


def set_store_policy(policy: "str | tuple[int, int, int, int]") -> None:
    """Process-wide, like the options it sets; takes effect with the next launch."""
    values = STORE_POLICIES[policy] if isinstance(policy, str) else tuple(policy)
    if len(values) != len(_STORE_POLICY_OPTIONS):
        raise ValueError(f"a store policy has {len(_STORE_POLICY_OPTIONS)} entries, got {values}")
    for option, value in zip(_STORE_POLICY_OPTIONS, values):
        set_option(option, value)


def get_store_policy() -> "tuple[int, int, int, int]":
    return tuple(get_option(option) for option in _STORE_POLICY_OPTIONS)
