"""The host-side tensor-list helper (yafsdp_amd/csrc/tensorlist.cpp) against the Python checks it
short-cuts: same pointer / mode arrays and dtype code for every list it accepts, and a hand-back to
the Python checks (which raise) for every list it does not."""

import numpy as np
import pytest
import torch

from yafsdp_amd import _native

tl = pytest.importorskip("yafsdp_amd._tensorlist")


def _table(numels, device="cpu"):
    """A TensorTable without its device-side half: only the host arrays ``_fill`` writes."""
    t = _native.TensorTable.__new__(_native.TensorTable)
    t.numels = list(numels)
    t.device = torch.device(device)
    t._init_host_arrays()
    return t


def _python_fill(table, tensors, modes):
    saved, _native._tensorlist = _native._tensorlist, None
    try:
        code = table._fill(tensors, modes, "tensors")
    finally:
        _native._tensorlist = saved
    return code, table._ptrs.copy(), table._modes.copy()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_modes", [False, True])
def test_same_arrays_as_the_python_checks(dtype, with_modes):
    rng = np.random.default_rng(5)
    numels = [int(x) for x in rng.integers(1, 300, 57)]
    tensors = [torch.empty(n, dtype=dtype) for n in numels]
    tensors[3] = tensors[40] = None
    modes = [int(x) for x in rng.integers(0, 3, len(numels))] if with_modes else None
    table = _table(numels)
    want = _python_fill(table, tensors, modes)
    table._ptrs[:] = 7
    table._modes[:] = 9
    code = table._fill(tensors, modes, "tensors")
    assert code == want[0] == _native.DTYPE_CODE[dtype]
    assert np.array_equal(table._ptrs, want[1]) and np.array_equal(table._modes, want[2])
    direct = tl.fill(tensors, modes, table._numels_arr.ctypes.data, table._ptrs.ctypes.data, table._modes.ctypes.data, False, -1)
    assert direct == code
    assert table._ptrs[3] == 0 and table._modes[3] == _native.MODE_SKIP


def test_all_skipped_and_tuple_input():
    table = _table([4, 5])
    assert table._fill((None, None), None, "tensors") == -1
    assert table._ptrs[:2].tolist() == [0, 0]
    assert table._fill((torch.empty(4), torch.empty(5)), [0, 0], "tensors") == -1


@pytest.mark.parametrize("case,error", [
    ("numel", ValueError), ("dtype_mix", TypeError), ("dtype_unsupported", TypeError),
    ("strided", (NotImplementedError, RuntimeError)),  # on a CPU tensor the device check of the error path fires first
    ("not_a_tensor", Exception),
])
def test_rejected_lists_raise_from_the_python_checks(case, error):
    numels = [6, 8]
    tensors = [torch.empty(6), torch.empty(8)]
    if case == "numel":
        tensors[1] = torch.empty(9)
    elif case == "dtype_mix":
        tensors[1] = torch.empty(8, dtype=torch.bfloat16)
    elif case == "dtype_unsupported":
        tensors = [torch.empty(6, dtype=torch.float64), torch.empty(8, dtype=torch.float64)]
    elif case == "strided":
        tensors[1] = torch.empty(4, 4).t()[:, :2]
    elif case == "not_a_tensor":
        tensors[1] = np.zeros(8, dtype=np.float32)
    table = _table(numels)
    args = (table._numels_arr.ctypes.data, table._ptrs.ctypes.data, table._modes.ctypes.data, False, -1)
    assert tl.fill(tensors, None, *args) == tl.REJECTED
    with pytest.raises(error):
        table._fill(tensors, None, "tensors")


def test_wrong_device_is_rejected():
    table = _table([4], device="cuda:0")  # no GPU needed: the CPU tensor is simply not on it
    args = (table._numels_arr.ctypes.data, table._ptrs.ctypes.data, table._modes.ctypes.data, True, 0)
    assert tl.fill([torch.empty(4)], None, *args) == tl.REJECTED
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        table._fill([torch.empty(4)], None, "tensors")


def test_bad_modes_are_handed_back():
    table = _table([4])
    args = (table._numels_arr.ctypes.data, table._ptrs.ctypes.data, table._modes.ctypes.data, False, -1)
    assert tl.fill([torch.empty(4)], [7], *args) == tl.REJECTED
    assert tl.fill([torch.empty(4)], [1, 1], *args) == tl.REJECTED
    assert tl.fill([torch.empty(4)], ["x"], *args) == tl.REJECTED


def test_all_contiguous():
    a, b = torch.empty(4, 4), torch.empty(4, 4).t()
    assert _native.all_contiguous([a, None, a]) and not _native.all_contiguous([a, b])
    assert tl.all_contiguous((a,)) and not tl.all_contiguous([None, b])
    with pytest.raises(TypeError):
        tl.all_contiguous([1])


def test_helper_is_faster_for_a_large_table():
    import time

    numels = [64] * 2000
    tensors = [torch.empty(64) for _ in numels]
    table = _table(numels)

    def clock(fn, reps=20):
        fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    fast = clock(lambda: table._fill(tensors, None, "tensors"))
    slow = clock(lambda: _python_fill(table, tensors, None))
    assert fast < slow / 3, (fast, slow)
