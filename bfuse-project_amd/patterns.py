"""Fusion index maps through the C ABI (host arithmetic of csrc/dispatch.h).

Counterpart of the reference's pattern generators, horizontal-fuser/src/Algorithms.cc.
"""
import ctypes as C
from dataclasses import dataclass
from typing import List, Sequence, Tuple

import numpy as np

from . import _lib

PATTERNS = {"zigzag": 0, "proportional": 1, "chunked": 2, "ranges": 3}


@dataclass
class LaunchDims:
    """GridDim / BlockDim of one kernel (horizontal-fuser/include/fuse/Contexts.h:13-26)."""
    grid: Tuple[int, int, int]
    block: Tuple[int, int, int]


def _dims_array(kernels: Sequence[LaunchDims]):
    arr = (_lib.LaunchDimsC * len(kernels))()
    for i, k in enumerate(kernels):
        arr[i].grid[:] = list(k.grid)
        arr[i].block[:] = list(k.block)
    return arr


class ThreadPlan:
    """hfusePattern (Algorithms.cc:19-116)."""

    def __init__(self, c):
        self.c = c
        n = c.n_kernels
        self.thr_lo = list(c.thr_lo[:n])
        self.thr_hi = list(c.thr_hi[:n])
        self.blocks = list(c.blocks[:n])
        self.fused_grid = c.fused_grid
        self.fused_block = c.fused_block

    def map(self, bid: int, tid: int):
        local = C.c_int(-1)
        k = _lib.lib().bfuse_map_thread(C.byref(self.c), bid, tid, C.byref(local))
        return k, local.value


class BlockPlan:
    """A block-fusion dispatch table (Algorithms.cc:118-739 lowered to segments)."""

    def __init__(self, c):
        self.c = c
        self.fused_grid = c.fused_grid
        self.fused_block = c.fused_block

    def map(self, bid: int):
        virt = C.c_int(-1)
        k = _lib.lib().bfuse_map_block(C.byref(self.c), bid, C.byref(virt))
        return k, virt.value

    def table(self, lo=0, hi=None):
        hi = self.fused_grid if hi is None else hi
        ks = np.empty(hi - lo, np.int32)
        vs = np.empty(hi - lo, np.int32)
        f = _lib.lib().bfuse_map_block
        virt = C.c_int()
        for i, b in enumerate(range(lo, hi)):
            ks[i] = f(C.byref(self.c), b, C.byref(virt))
            vs[i] = virt.value
        return ks, vs

    def table_device(self, lo=0, hi=None):
        """The same table evaluated by the device build of the map (needs a GPU)."""
        hi = self.fused_grid if hi is None else hi
        ks = np.empty(hi - lo, np.int32)
        vs = np.empty(hi - lo, np.int32)
        _lib.check(_lib.lib().bfuse_map_blocks_device(C.byref(self.c), lo, hi, ks.ctypes.data, vs.ctypes.data))
        return ks, vs

    def table_device_noalloc(self, lo=0, hi=None):
        """table_device through the entry point that allocates nothing (fixed staging array,
        at most BFUSE_NOALLOC_MAX_IDS = 262144 ids per call)."""
        hi = self.fused_grid if hi is None else hi
        ks = np.empty(max(hi - lo, 0), np.int32)
        vs = np.empty(max(hi - lo, 0), np.int32)
        _lib.check(_lib.lib().bfuse_map_blocks_device_noalloc(C.byref(self.c), lo, hi, ks.ctypes.data, vs.ctypes.data))
        return ks, vs

    def segments(self) -> List[dict]:
        out = []
        for s in self.c.seg[: self.c.n_seg]:
            out.append({"lo": s.lo, "hi": s.hi, "period": s.period,
                        "slots": [(sl.kern, sl.off, sl.width, sl.base) for sl in s.slot[: s.n_slot]]})
        return out


def plan_threads(kernels: Sequence[LaunchDims], pad: int = 64) -> ThreadPlan:
    out = _lib.ThreadPlanC()
    _lib.check(_lib.lib().bfuse_plan_threads(len(kernels), _dims_array(kernels), pad, C.byref(out)))
    return ThreadPlan(out)


def plan_blocks(pattern: str, kernels: Sequence[LaunchDims], p0: int = 1, p1: int = 1) -> BlockPlan:
    out = _lib.BlockPlanC()
    _lib.check(_lib.lib().bfuse_plan_blocks(PATTERNS[pattern], len(kernels), _dims_array(kernels), p0, p1, C.byref(out)))
    return BlockPlan(out)
