"""Tables with more than 16 tensors pass the per-call tensor pointers and modes through staging slots inside the
table.  A call with the arrays of an earlier call reuses that call's device copy; a call with new arrays stages
them; neither waits on the host, and when every slot belongs to a queued call the C entry point says so instead
of waiting."""

import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_bits_equal, mixed_values
from oracle import torch_ops

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _want(numels, t_pad, grads, modes, old, pre):
    want = old.clone()
    views = list(want[: sum(numels)].split(numels))
    cp = [i for i, m in enumerate(modes) if m == 1]
    ad = [i for i, m in enumerate(modes) if m == 2]
    torch_ops.reduce_copy_in([views[i] for i in cp], [grads[i] for i in cp], False)
    torch_ops.reduce_copy_in([views[i] for i in ad], [grads[i] for i in ad], True)
    want[sum(numels):t_pad] = 0
    torch_ops.div_if_needed(want[:t_pad], pre)
    return want


def test_unchanged_and_changed_pointer_sets_alternate():
    from yafsdp_amd import _native as nat

    rng = np.random.default_rng(7)
    g = torch.Generator().manual_seed(7)
    p = 40
    numels = (np.floor(np.exp2(rng.uniform(0, 12, size=p))).astype(np.int64) | 1).tolist()
    t, t_pad = sum(numels), sum(numels) + 77
    table = nat.TensorTable(numels, t_pad, DEV)
    # three tensor sets with different values, each at addresses of its own; set A is used again and again
    sets = [[mixed_values(g, n, torch.bfloat16, 1e-3) for n in numels] for _ in range(3)]
    dsets = [[x.to(DEV) for x in s] for s in sets]
    old = mixed_values(g, t_pad, torch.float32, 1e-3)
    mode_sets = [[1] * p, rng.integers(0, 3, size=p).tolist(), rng.integers(1, 3, size=p).tolist()]
    outs_want = [mixed_values(g, n, torch.float32, 1.0) for n in numels]  # scatter-out source data is `old`
    order = [0, 0, 1, 0, 2, 2, 0, 1, 1, 0, 0]
    for step, k in enumerate(order):
        modes = mode_sets[(step + k) % 3]
        got = old.to(DEV)
        table.gather_in(dsets[k], got, modes, 8.0, zero_pad=True)
        # a scatter-out through the same table in between: it shares the staging slots
        douts = [torch.empty(n, dtype=torch.float32, device=DEV) for n in numels]
        table.scatter_out(old.to(DEV), douts)
        assert_bits_equal(got, _want(numels, t_pad, sets[k], modes, old, 8.0), f"step {step}: set {k}")
        for d, w in zip(douts, old[:t].split(numels)):
            assert_bits_equal(d, w, f"step {step}: copy-out")
    # same pointers, different values: the cached slot holds pointers, not data
    for x in dsets[0]:
        x.mul_(-2.0)
    new_vals = [x.cpu() for x in dsets[0]]
    got = old.to(DEV)
    table.gather_in(dsets[0], got, mode_sets[0], None, zero_pad=True)
    assert_bits_equal(got, _want(numels, t_pad, new_vals, mode_sets[0], old, None), "same pointers, new values")
    # same pointers, different modes: a different staged set
    got = old.to(DEV)
    table.gather_in(dsets[0], got, mode_sets[1], None, zero_pad=True)
    assert_bits_equal(got, _want(numels, t_pad, new_vals, mode_sets[1], old, None), "same pointers, new modes")
    torch.cuda.synchronize()
    table.close()
    del outs_want


def test_many_queued_calls_with_new_pointers_never_mix_their_sets():
    """More different tensor sets in flight than the table has slots: the binding waits for the stream when the
    library reports that every slot is taken; every call still sees its own pointers."""
    from yafsdp_amd import _native as nat

    g = torch.Generator().manual_seed(11)
    p = 24
    numels = [3001 + 2 * i for i in range(p)]
    t = sum(numels)
    table = nat.TensorTable(numels, t, DEV)
    big_a = torch.empty(64 << 20, dtype=torch.float32, device=DEV)
    big_b = torch.empty_like(big_a)
    sets = [[mixed_values(g, n, torch.bfloat16, 1e-3, specials=False) for n in numels] for _ in range(20)]
    dsets = [[x.to(DEV) for x in s] for s in sets]
    flats = [torch.zeros(t, dtype=torch.bfloat16, device=DEV) for _ in sets]
    torch.cuda.synchronize()
    for _ in range(4):
        nat.flat_copy(big_b, big_a)  # about a millisecond of queued work in front of the table calls
    for d, f in zip(dsets, flats):
        table.gather_in(d, f)
    torch.cuda.synchronize()
    for s, f in zip(sets, flats):
        assert_bits_equal(f, torch.cat(s), "queued gather_in")
    table.close()


def test_c_entry_point_reports_busy_instead_of_waiting():
    from yafsdp_amd import _native as nat

    lib = nat.lib
    p = 20
    numels = [1000 + i for i in range(p)]
    t = sum(numels)
    table = nat.TensorTable(numels, t, DEV)
    sets = [[torch.ones(n, dtype=torch.bfloat16, device=DEV) * (k + 1) for n in numels] for k in range(10)]
    flats = [torch.zeros(t, dtype=torch.bfloat16, device=DEV) for _ in sets]
    big_a = torch.empty(128 << 20, dtype=torch.float32, device=DEV)
    big_b = torch.empty_like(big_a)
    stream = ctypes.c_void_p(torch.cuda.current_stream(DEV).cuda_stream)
    torch.cuda.synchronize()
    codes = []
    with torch.cuda.device(DEV):
        for _ in range(8):
            nat.flat_copy(big_b, big_a)  # several milliseconds of queued work: nothing behind it finishes meanwhile
        for d, f in zip(sets, flats):
            ptrs = np.array([x.data_ptr() for x in d], dtype=np.uint64)
            codes.append(lib.yafsdp_gather_in(table._handle, ptrs.ctypes.data, None, 1, f.data_ptr(), 1, 0.0, 1, stream))
    torch.cuda.synchronize()
    assert codes[:8] == [0] * 8, codes
    assert codes[8:] == [-7, -7], codes
    assert b"staging slot" in lib.yafsdp_error_string(-7)
    for k, f in enumerate(flats):
        expect = float(k + 1) if codes[k] == 0 else 0.0  # a refused call enqueues nothing
        assert float(f.float().min()) == expect and float(f.float().max()) == expect
    # once the queue has drained the slots are free again
    with torch.cuda.device(DEV):
        ptrs = np.array([x.data_ptr() for x in sets[9]], dtype=np.uint64)
        assert lib.yafsdp_gather_in(table._handle, ptrs.ctypes.data, None, 1, flats[9].data_ptr(), 1, 0.0, 1, stream) == 0
    torch.cuda.synchronize()
    assert float(flats[9].float().min()) == 10.0
    table.close()
