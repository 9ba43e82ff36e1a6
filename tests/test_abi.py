"""The C-ABI library loads without a GPU and exports every symbol that
include/yafsdp_hip.h declares (no compute calls here)."""

import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "yafsdp_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(yafsdp_[a-z_]+)\s*\(", text)))


def test_header_and_binding_agree():
    from yafsdp_amd import _native

    declared = _declared_functions()
    assert declared, "no declarations parsed"
    assert sorted(_native.EXPORTED_SYMBOLS) == declared


def test_library_exports_every_symbol():
    from yafsdp_amd import _native

    for name in _declared_functions():
        assert hasattr(_native.lib, name), name
    import __graft_entry__

    assert _native.lib.yafsdp_version() // 1000 == __graft_entry__.ABI_MAJOR  # what build() checks
    assert _native.lib.yafsdp_version() == 1007  # 1.1: yafsdp_flat_copy_bytes; 1.2-1.5: the four write-through tail options; 1.6: per-table tails, pre-multiplied share; 1.7: pre-multiplied fan-in
    assert _native.error_string(0) == "success"
    assert "dtype" in _native.error_string(-2)


def test_argument_validation_without_gpu():
    """Entry points reject bad arguments before touching the device."""
    from yafsdp_amd import _native

    L = _native.lib
    assert L.yafsdp_flat_copy(None, 9, None, 0, 4, None) == -2
    assert L.yafsdp_flat_copy(None, 0, None, 0, -1, None) == -1
    assert L.yafsdp_flat_copy(None, 0, None, 0, 4, None) == -1
    assert L.yafsdp_flat_copy(None, 0, None, 0, 0, None) == 0
    assert L.yafsdp_flat_div(None, 0, 0, 8.0, None) == 0
    assert L.yafsdp_post_reduce(None, 0, None, 5, 0, 0.0, 0, None) == -2
    # empty ranges are fine whatever their pointers (torch hands out null for empty tensors)
    assert L.yafsdp_post_reduce(None, 1, None, 0, 0, 8.0, 1, None) == 0
    assert L.yafsdp_flat_div_copy(None, 1, None, 0, 0, 3.0, None) == 0
    assert L.yafsdp_flat_premul(None, 1, 0, 1.0 / 3, None) == 0
    assert L.yafsdp_flat_premul(None, 7, 0, 0.5, None) == -2
    assert L.yafsdp_flat_premul(None, 1, 4, 0.5, None) == -1
    assert L.yafsdp_flat_premul(None, 1, 0, float("inf"), None) == -1  # no finite scalar in the data type
    assert L.yafsdp_post_reduce_premul(None, 0, None, 1, 0, 0.2, 1, None) == 0
    assert L.yafsdp_post_reduce_premul(None, 0, None, 1, 4, 0.2, 1, None) == -1
    assert L.yafsdp_table_set_option(None, 4, 64) == -1
    assert L.yafsdp_set_option(99, 1) == -1
    assert L.yafsdp_set_option(0, 0) == -1
    assert L.yafsdp_set_option(2, 63) == -1
    assert L.yafsdp_set_option(2, 28) == 0
    assert L.yafsdp_set_option(3, 3) == -1
    assert L.yafsdp_set_option(3, 0) == 0
    assert L.yafsdp_set_option(4, -1) == -1
    assert L.yafsdp_set_option(4, (1 << 20) + 1) == -1
    tail = ctypes.c_int(-1)
    assert L.yafsdp_get_option(4, ctypes.byref(tail)) == 0 and tail.value == 64
    assert L.yafsdp_set_option(4, 0) == 0 and L.yafsdp_get_option(4, ctypes.byref(tail)) == 0 and tail.value == 0
    assert L.yafsdp_set_option(4, 64) == 0
    assert L.yafsdp_set_option(5, -1) == -1
    assert L.yafsdp_get_option(5, ctypes.byref(tail)) == 0 and tail.value == 0
    assert L.yafsdp_set_option(5, 7) == 0 and L.yafsdp_get_option(5, ctypes.byref(tail)) == 0 and tail.value == 7
    assert L.yafsdp_set_option(5, 0) == 0
    assert L.yafsdp_get_option(6, ctypes.byref(tail)) == 0 and tail.value == 0
    assert L.yafsdp_set_option(6, 1 << 20) == 0 and L.yafsdp_get_option(6, ctypes.byref(tail)) == 0 and tail.value == 1 << 20
    assert L.yafsdp_set_option(6, 0) == 0
    assert L.yafsdp_get_option(7, ctypes.byref(tail)) == 0 and tail.value == 0
    assert L.yafsdp_set_option(7, 5) == 0 and L.yafsdp_get_option(7, ctypes.byref(tail)) == 0 and tail.value == 5
    assert L.yafsdp_set_option(7, 0) == 0
    assert L.yafsdp_set_option(8, 1) == -1
    assert L.yafsdp_gather_in(None, None, None, 0, None, 0, 0.0, 1, None) == -1
    assert L.yafsdp_table_destroy(None) == 0
    # operands that overlap without being the same buffer are refused (addresses are never dereferenced here)
    assert L.yafsdp_flat_copy(0x10000, 1, 0x10008, 1, 64, None) == -1          # shifted by 4 elements
    assert L.yafsdp_flat_copy(0x10000, 1, 0x10000, 0, 64, None) == -1          # same base, 2-byte over 4-byte elements
    assert L.yafsdp_post_reduce(0x10000, 0, 0x100f0, 1, 64, 0.0, 1, None) == -1  # chunk inside the shard
    assert L.yafsdp_flat_copy(0x10000, 1, 0x10000, 1, 64, None) == 0           # self-copy: nothing to do
    # opaque bytes: same rules at byte granularity
    assert L.yafsdp_flat_copy_bytes(None, None, -1, None) == -1
    assert L.yafsdp_flat_copy_bytes(None, None, 8, None) == -1
    assert L.yafsdp_flat_copy_bytes(None, None, 0, None) == 0
    assert L.yafsdp_flat_copy_bytes(0x10001, 0x10001, 63, None) == 0             # self-copy
    assert L.yafsdp_flat_copy_bytes(0x10001, 0x10004, 63, None) == -1            # odd addresses, overlapping
    assert L.yafsdp_flat_copy_bytes(0x10000, 0x10008, 64, None) == -1            # even addresses, overlapping
    # element counts that cannot be a real buffer are refused at table creation

    import numpy as np

    handle = ctypes.c_void_p()
    huge = np.array([1 << 61, 1 << 61], dtype=np.int64)
    assert L.yafsdp_table_create(2, huge.ctypes.data, 1 << 62, ctypes.byref(handle)) == -1
    neg = np.array([4, -1], dtype=np.int64)
    assert L.yafsdp_table_create(2, neg.ctypes.data, 8, ctypes.byref(handle)) == -1


def test_no_product_module_imports_the_oracle():
    pkg = os.path.join(ROOT, "yafsdp_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hip.h", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", src, flags=re.M), f
                assert "libbufpath_ref" not in src, f


def test_store_policies_set_the_four_tail_options():
    import pytest

    from yafsdp_amd import _native

    # the library's own defaults are the cache-neutral policy; the one tuned to a loop over one buffer set is opt-in
    assert _native.get_store_policy() == _native.STORE_POLICIES["rotating_sets"] == (0, 0, 0, 64)
    try:
        _native.set_store_policy("single_set")
        assert _native.get_store_policy() == (1 << 20, 1 << 20, 0, 96)
        assert _native.get_option(_native.OPT_GATHER_TAIL_MB) == 96
        _native.set_store_policy((5, 6, 7, 8))
        assert _native.get_store_policy() == (5, 6, 7, 8)
        with pytest.raises(KeyError):
            _native.set_store_policy("no_such_policy")
        with pytest.raises(ValueError):
            _native.set_store_policy((1, 2, 3))
    finally:
        _native.set_store_policy("rotating_sets")
