"""The entry point that allocates nothing (bfuse_map_blocks_device_noalloc) against the entry point
it is a variant of (bfuse_map_blocks_device), through the C ABI, on the GPU.

Index work: the two must agree exactly.  Two calls in a row, the second with a smaller input, so
that contents the fixed staging array keeps from the first call would show in the second; then a
range that ends inside the array, the largest range the array holds, and one past it (refused).
"""
import ctypes as C

import numpy as np
import pytest

import bfuse_project_amd as bf
from bfuse_project_amd import _lib
from bfuse_project_amd._lib import BfuseError

pytestmark = pytest.mark.gpu

MAX_IDS = 262144   # BFUSE_NOALLOC_MAX_IDS


def _plan(pattern, params, grids):
    return bf.plan_blocks(pattern, [bf.LaunchDims((g, 1, 1), (64, 1, 1)) for g in grids], *params)


def test_noalloc_entry_point_equals_the_allocating_one_on_two_calls_in_a_row():
    _lib.check(_lib.lib().bfuse_init(0))
    big = _plan("zigzag", (4, 1), (65536, 1858560))      # a reference golden: ratio 4:1, 1.9 M fused blocks
    small = _plan("chunked", (84, 1), (1024, 1815))      # the reference's SM-chunk golden, 2839 fused blocks
    print("[noalloc] first call: 200000 ids of the 4:1 zig-zag, from 300000", flush=True)
    k_ref, v_ref = big.table_device(300000, 500000)
    k_new, v_new = big.table_device_noalloc(300000, 500000)
    assert np.array_equal(k_new, k_ref) and np.array_equal(v_new, v_ref)
    print("[noalloc] second call, smaller: the whole chunk-84 grid", flush=True)
    k_ref, v_ref = small.table_device()
    k_new, v_new = small.table_device_noalloc()
    assert k_new.size == 2839
    assert np.array_equal(k_new, k_ref) and np.array_equal(v_new, v_ref)
    # and against the host evaluation of the same plan
    k_host, v_host = small.table()
    assert np.array_equal(k_new, k_host) and np.array_equal(v_new, v_host)


def test_noalloc_entry_point_limits():
    _lib.check(_lib.lib().bfuse_init(0))
    big = _plan("zigzag", (1, 1), (384, 100352 * 4))
    print("[noalloc] the largest range the staging array holds", flush=True)
    k_new, v_new = big.table_device_noalloc(7, 7 + MAX_IDS)
    k_ref, v_ref = big.table_device(7, 7 + MAX_IDS)
    assert np.array_equal(k_new, k_ref) and np.array_equal(v_new, v_ref)
    print("[noalloc] one id more is refused before anything is launched", flush=True)
    with pytest.raises(BfuseError, match="fixed staging array holds 262144"):
        big.table_device_noalloc(0, MAX_IDS + 1)
    with pytest.raises(BfuseError):
        big.table_device_noalloc(5, 5)          # empty range, as the allocating entry point
    # a refused call leaves the entry point usable
    k_new, v_new = big.table_device_noalloc(0, 1000)
    k_host, v_host = big.table(0, 1000)
    assert np.array_equal(k_new, k_host) and np.array_equal(v_new, v_host)


def test_noalloc_entry_point_leaves_free_device_memory_unchanged():
    """Free device memory as the runtime reports it, before and after repeated calls (one call first, so
    that whatever the first launch of the kernel loads is already there)."""
    l = _lib.lib()
    _lib.check(l.bfuse_init(0))
    plan = _plan("zigzag", (4, 1), (65536, 1858560))
    plan.table_device_noalloc(0, MAX_IDS)
    before = C.c_size_t()
    _lib.check(l.bfuse_device_memory(C.byref(before), None))
    for lo in (0, 1000, 500000):
        plan.table_device_noalloc(lo, lo + MAX_IDS)
        plan.table_device_noalloc(lo, lo + 77)
    after = C.c_size_t()
    _lib.check(l.bfuse_device_memory(C.byref(after), None))
    print(f"[noalloc] free device memory {before.value} -> {after.value} bytes", flush=True)
    assert after.value == before.value
