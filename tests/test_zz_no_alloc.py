"""The entry point that allocates nothing (``yafsdp_flat_sumsq_static``) against the entry point it is a variant of
(``yafsdp_flat_sumsq`` with a caller-provided workspace), called through the C ABI."""

import ctypes
import gc

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")


def _sumsq_pair(lib, src, accumulate, start):
    """(workspace entry point, static entry point) on the same input; both outputs start at `start`."""
    dt = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[src.dtype]
    stream = ctypes.c_void_p(torch.cuda.current_stream(DEV).cuda_stream)
    want = torch.full((1,), start, dtype=torch.float64, device=DEV)
    got = torch.full((1,), start, dtype=torch.float64, device=DEV)
    nbytes = lib.yafsdp_sumsq_workspace_bytes()
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    rc = lib.yafsdp_flat_sumsq(src.data_ptr(), dt, src.numel(), want.data_ptr(), int(accumulate), workspace.data_ptr(),
                               nbytes, stream)
    assert rc == 0, lib.yafsdp_error_string(rc)
    torch.cuda.synchronize()
    # (no garbage of earlier tests may be collected, and its device memory returned, between the two readings)
    gc.collect()
    gc.disable()
    try:
        # the driver's own count of free device memory sees a hipMalloc inside the library; torch's statistics
        # (its caching allocator's) would not
        before_free, _ = torch.cuda.mem_get_info(DEV)
        before = torch.cuda.memory_allocated(DEV)
        rc = lib.yafsdp_flat_sumsq_static(src.data_ptr(), dt, src.numel(), got.data_ptr(), int(accumulate), stream)
        assert rc == 0, lib.yafsdp_error_string(rc)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(DEV) == before
        assert torch.cuda.mem_get_info(DEV)[0] == before_free
    finally:
        gc.enable()
    return want, got


def test_static_scratch_entry_point_matches_the_workspace_one():
    from yafsdp_amd import _native

    lib = _native.lib
    g = torch.Generator().manual_seed(77)
    big = (torch.randn(3_000_001, generator=g) * 1e-2).to(DEV)
    small = (torch.randn(70_003, generator=g) * 3.0).bfloat16().to(DEV)
    with torch.cuda.device(DEV):
        # the first call on a device performs the set-up (the scratch's address is looked up): before the
        # readings of free memory below, which the first use of a code object may move
        assert lib.yafsdp_flat_sumsq_static(None, 0, 0, None, 0, None) == 0
        _sumsq_pair(lib, small[:64], False, 0.0)
        # two calls in a row, the second with a smaller input of another dtype: whatever the first call left in
        # the shared scratch must not leak into the second
        want, got = _sumsq_pair(lib, big, False, 123.0)
        assert torch.equal(want.view(torch.int64), got.view(torch.int64))
        assert abs(float(got) - float((big.double() ** 2).sum())) <= 1e-9 * float(got)
        want, got = _sumsq_pair(lib, small, False, -5.0)
        assert torch.equal(want.view(torch.int64), got.view(torch.int64))
        assert abs(float(got) - float((small.double() ** 2).sum())) <= 1e-9 * float(got)
        # accumulating form, on an unaligned start, then a tiny input
        want, got = _sumsq_pair(lib, big[3:1_000_000], True, 0.5)
        assert torch.equal(want.view(torch.int64), got.view(torch.int64))
        want, got = _sumsq_pair(lib, small[:5], True, 0.5)
        assert torch.equal(want.view(torch.int64), got.view(torch.int64))
        # nothing to add: the output becomes 0, or keeps its value when accumulating, from both entry points
        want, got = _sumsq_pair(lib, small[:0], False, 7.0)
        assert float(want) == 0.0 and float(got) == 0.0
        want, got = _sumsq_pair(lib, small[:0], True, 7.0)
        assert float(want) == 7.0 and float(got) == 7.0


def test_static_scratch_entry_point_limits():
    from yafsdp_amd import _native

    lib = _native.lib
    limit = lib.yafsdp_flat_sumsq_static_max_numel()
    assert limit == 1 << 31
    out = torch.zeros(1, dtype=torch.float64, device=DEV)
    x = torch.ones(8, device=DEV)
    with torch.cuda.device(DEV):
        # beyond the limit: refused before anything is launched or read
        rc = lib.yafsdp_flat_sumsq_static(x.data_ptr(), 0, limit + 1, out.data_ptr(), 0, None)
        assert rc == -6 and b"2^31" in lib.yafsdp_error_string(rc)
        assert lib.yafsdp_flat_sumsq_static(x.data_ptr(), 7, 8, out.data_ptr(), 0, None) == -2
        assert lib.yafsdp_flat_sumsq_static(None, 0, 8, out.data_ptr(), 0, None) == -1
        # n == 0 only performs the set-up
        assert lib.yafsdp_flat_sumsq_static(None, 0, 0, None, 0, None) == 0
        _native.flat_sumsq_static(x, out)
        torch.cuda.synchronize()
    assert float(out) == 8.0
