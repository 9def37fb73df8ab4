"""Host-side mirror of the reference harness (test-utils/test-suite-files/operation_h.py:9-27,
operation_cu.py:123-256): initialize / run_kernel1 / run_kernel2 / run_parallel / run_fuse /
finalize over numpy buffers, plus the device-resident launch and GPU-side timing entry points.
"""
import ctypes as C
import os
from dataclasses import dataclass, replace
from typing import List, Optional, Sequence

import numpy as np

from . import _lib

MODES = {"kernel1": 0, "kernel2": 1, "parallel": 2, "hfuse": 3, "bfuse": 4, "serial": 5}


@dataclass
class KernelHandle:
    name: str
    func: int
    kind: int                 # 0 single, 1 bfuse, 2 hfuse, 3 bfuse with a run-time plan (persistent workgroups)
    grid: tuple
    block: tuple
    has_barriers: bool
    regs: int
    lds_bytes: int
    shapes: tuple             # ((4 ints) x 3) for single kernels
    elem_bytes: tuple
    sides: tuple
    pattern: int
    p0: int
    p1: int
    n_sides: int = 2          # kernels a fused kernel runs (1 for a standalone kernel)
    matrix: bool = False      # standalone kernel whose inner loop is a stream of MFMAs (GEMMs, convolutions)


def _handle(ci: "_lib.KernelInfoC") -> KernelHandle:
    return KernelHandle(ci.name.decode(), ci.func, ci.kind, tuple(ci.grid), tuple(ci.block), bool(ci.has_barriers),
                        ci.regs, ci.lds_bytes, tuple(tuple(s) for s in ci.shape), tuple(ci.elem_bytes),
                        tuple([ci.side[0].value.decode(), ci.side[1].value.decode()] +
                              [ci.side_more[i].value.decode() for i in range(max(0, ci.n_sides - 2))]),
                        ci.pattern, ci.p0, ci.p1, ci.n_sides, bool(ci.matrix_cores))


def kernel_info(name: str) -> KernelHandle:
    ci = _lib.KernelInfoC()
    _lib.check(_lib.lib().bfuse_kernel_find(name.encode(), C.byref(ci)))
    return _handle(ci)


def list_kernels() -> List[KernelHandle]:
    l = _lib.lib()
    out = []
    n = l.bfuse_kernel_count()
    if n == 0:      # the library always holds kernels: an empty registry means a module named in the environment did not load
        raise _lib.BfuseError(-1, l.bfuse_last_error().decode() or "the kernel registry is empty")
    for i in range(n):
        ci = _lib.KernelInfoC()
        _lib.check(l.bfuse_kernel_at(i, C.byref(ci)))
        out.append(_handle(ci))
    return out


def _i4(shape):
    s = list(shape) + [1] * (4 - len(shape))
    return (C.c_int * 4)(*s)


def _u3(v):
    return (C.c_uint * 3)(*v)


_DT = {4: np.float32, 2: np.uint16, 1: np.uint8}


class Operation:
    """One pair of sides with their device buffers (the reference keeps them in file-scope
    globals; so does the library -- one Operation may be live at a time)."""

    def __init__(self, k1: str, k2: str, device: int = 0):
        self.l = _lib.lib()
        _lib.check(self.l.bfuse_init(device))
        self.k = [kernel_info(k1), kernel_info(k2)]
        for side, k in enumerate(self.k, 1):
            if k.kind != 0:
                raise ValueError(f"{k.name} is a fused kernel; sides must be standalone kernels")
            _lib.check(self.l.bfuse_set_elem_bytes(side, *k.elem_bytes))
        self.shapes = [[_i4(s) for s in k.shapes] for k in self.k]
        _lib.check(self.l.initialize_kernel1(*self.shapes[0]))
        try:
            _lib.check(self.l.initialize_kernel2(*self.shapes[1]))
        except Exception:
            self.l.finalize_kernel1()
            raise
        self.live = True

    # -- context management ------------------------------------------------------------
    def close(self):
        if self.live:
            self.live = False
            _lib.check(self.l.finalize_kernel1())
            _lib.check(self.l.finalize_kernel2())

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- helpers -----------------------------------------------------------------------
    def _host(self, side, idx, arr):
        k = self.k[side]
        dt = _DT[k.elem_bytes[idx]]
        a = np.ascontiguousarray(arr, dtype=dt)
        want = int(np.prod(k.shapes[idx]))
        if a.size != want:
            raise ValueError(f"{k.name}: tensor {idx} has {a.size} elements, kernel expects {want}")
        return a

    def empty_output(self, side):
        k = self.k[side]
        return np.empty(tuple(d for d in k.shapes[2]), _DT[k.elem_bytes[2]])

    def fused(self, kind: str, suffix: str = "") -> KernelHandle:
        return kernel_info(f"{self.k[0].name}_{self.k[1].name}_fused_{kind}{suffix}")

    def fused_rt(self) -> KernelHandle:
        """The block-fused kernel of this pair whose dispatch plan is set at run time."""
        return kernel_info(f"{self.k[0].name}_{self.k[1].name}_fused_bfuse_rt")

    def set_plan(self, fused: KernelHandle, plan, workgroups: Optional[int] = None) -> KernelHandle:
        """Installs `plan` (patterns.BlockPlan) in a run-time-plan kernel and returns the handle to
        launch it with: the plan's fused grid, or `workgroups` persistent workgroups striding over it."""
        _lib.check(self.l.bfuse_set_plan(fused.func, C.byref(plan.c)))
        n = plan.fused_grid if workgroups is None else min(int(workgroups), plan.fused_grid)
        return replace(fused, grid=(n, 1, 1))

    # -- operation.h mirror (H2D, launch, sync, D2H) ---------------------------------------
    def run_kernel(self, side: int, I, F) -> np.ndarray:
        k = self.k[side]
        I, F = self._host(side, 0, I), self._host(side, 1, F)
        O = self.empty_output(side)
        fn = self.l.run_kernel1 if side == 0 else self.l.run_kernel2
        _lib.check(fn(I.ctypes.data, F.ctypes.data, O.ctypes.data, *self.shapes[side], k.func, _u3(k.grid), _u3(k.block), side))
        return O

    def run_parallel(self, I1, F1, I2, F2):
        a, b = self.k
        I1, F1, I2, F2 = self._host(0, 0, I1), self._host(0, 1, F1), self._host(1, 0, I2), self._host(1, 1, F2)
        O1, O2 = self.empty_output(0), self.empty_output(1)
        _lib.check(self.l.run_parallel(I1.ctypes.data, F1.ctypes.data, O1.ctypes.data, I2.ctypes.data, F2.ctypes.data,
                                       O2.ctypes.data, *self.shapes[0], *self.shapes[1], a.func, b.func,
                                       _u3(a.grid), _u3(a.block), _u3(b.grid), _u3(b.block), 0, 0))
        return O1, O2

    def run_fuse(self, fused: KernelHandle, I1, F1, I2, F2):
        I1, F1, I2, F2 = self._host(0, 0, I1), self._host(0, 1, F1), self._host(1, 0, I2), self._host(1, 1, F2)
        O1, O2 = self.empty_output(0), self.empty_output(1)
        _lib.check(self.l.run_fuse(I1.ctypes.data, F1.ctypes.data, O1.ctypes.data, I2.ctypes.data, F2.ctypes.data,
                                   O2.ctypes.data, *self.shapes[0], *self.shapes[1], fused.func,
                                   _u3(fused.grid), _u3(fused.block), 0, 0))
        return O1, O2

    # -- device-resident ---------------------------------------------------------------
    def upload(self, side: int, I, F):
        I, F = self._host(side, 0, I), self._host(side, 1, F)
        _lib.check(self.l.bfuse_upload(side + 1, I.ctypes.data, F.ctypes.data))

    def zero_outputs(self):
        _lib.check(self.l.bfuse_zero_output(1))
        _lib.check(self.l.bfuse_zero_output(2))

    def download(self, side: int) -> np.ndarray:
        O = self.empty_output(side)
        _lib.check(self.l.bfuse_download(side + 1, O.ctypes.data))
        return O

    def upload_part(self, side: int, tensor: int, offset: int, arr):
        """Writes `arr` into tensor 0 (I) or 1 (F) of the side, starting at element `offset`."""
        k = self.k[side]
        a = np.ascontiguousarray(arr, dtype=_DT[k.elem_bytes[tensor]])
        _lib.check(self.l.bfuse_upload_part(side + 1, tensor, offset * a.itemsize, a.ctypes.data, a.nbytes))

    def download_part(self, side: int, offset: int, count: int) -> np.ndarray:
        """`count` elements of the side's output, starting at element `offset`."""
        O = np.empty(count, _DT[self.k[side].elem_bytes[2]])
        _lib.check(self.l.bfuse_download_part(side + 1, offset * O.itemsize, O.ctypes.data, O.nbytes))
        return O

    def fill_uniform_device(self, side: int, tensor: int, seed: int, lo: float, hi: float):
        """Fills tensor 0 (I) or 1 (F) of the side in HBM with the values fill_uniform(seed, n, lo, hi) gives."""
        _lib.check(self.l.bfuse_fill_uniform_device(side + 1, tensor, seed, lo, hi))

    def checksum_output(self, side: int, chunk_elems: int) -> np.ndarray:
        """Device-side checksums of the side's output in chunks of `chunk_elems` elements: an array
        [chunks, 2] of uint64 that `checksum_of` reproduces on the host for expected contents."""
        k = self.k[side]
        total = int(np.prod(k.shapes[2]))
        if chunk_elems < 1 or total % chunk_elems:
            raise ValueError(f"{k.name}: chunks of {chunk_elems} elements do not divide the output's {total}")
        sums = np.zeros((total // chunk_elems, 2), np.uint64)
        _lib.check(self.l.bfuse_checksum_output(side + 1, chunk_elems * k.elem_bytes[2], sums.ctypes.data))
        return sums

    def _mode_args(self, mode: str, fused: Optional[KernelHandle]):
        a, b = self.k
        if mode == "kernel1":
            return (a.func, _u3(a.grid), _u3(a.block), None, None, None)
        if mode == "kernel2":
            return (b.func, _u3(b.grid), _u3(b.block), None, None, None)
        if mode in ("parallel", "serial"):
            return (a.func, _u3(a.grid), _u3(a.block), b.func, _u3(b.grid), _u3(b.block))
        if fused is None:
            raise ValueError("fused kernel handle required")
        return (fused.func, _u3(fused.grid), _u3(fused.block), None, None, None)

    def set_sync_spin_limit(self, kernel: KernelHandle, polls: int):
        """Polls a side barrier makes before it gives up, for every kernel of `kernel`'s module."""
        _lib.check(self.l.bfuse_set_sync_spin_limit(kernel.func, polls))

    def launch(self, mode: str, fused: Optional[KernelHandle] = None):
        _lib.check(self.l.bfuse_launch(MODES[mode], *self._mode_args(mode, fused)))

    def synchronize(self):
        _lib.check(self.l.bfuse_synchronize())

    def time(self, mode: str, fused: Optional[KernelHandle] = None, warmup: int = 3, reps: int = 30):
        """GPU-side microseconds per repetition: (total, kernel_a, kernel_b) arrays.  The default
        3 + 30 is the reference's sampling (scripts/profile_test_suite.py:10-11)."""
        tot, ta, tb = (np.zeros(reps, np.float32) for _ in range(3))
        fp = C.POINTER(C.c_float)
        _lib.check(self.l.bfuse_time(MODES[mode], *self._mode_args(mode, fused), warmup, reps,
                                     tot.ctypes.data_as(fp), ta.ctypes.data_as(fp), tb.ctypes.data_as(fp)))
        return tot, ta, tb

    def time_batched(self, mode: str, fused: Optional[KernelHandle] = None, warmup: int = 3, reps: int = 30) -> float:
        us = C.c_float()
        _lib.check(self.l.bfuse_time_batched(MODES[mode], *self._mode_args(mode, fused), warmup, reps, C.byref(us)))
        return us.value

    def time_graph(self, mode: str, fused: Optional[KernelHandle] = None, chain: int = 20, reps: int = 10) -> float:
        """Mean microseconds per repetition of `mode` when `chain` repetitions are captured into one HIP graph and
        the graph is replayed `reps` times ('serial': the two kernels as dependent nodes; 'parallel': as independent
        nodes between a fork and a join)."""
        us = C.c_float()
        _lib.check(self.l.bfuse_time_graph(MODES[mode], *self._mode_args(mode, fused), chain, reps, C.byref(us)))
        return us.value


class GroupOperation:
    """Two to four sides for fusions of more than two kernels (the reference's fuser takes a list of
    kernels, horizontal-fuser/src/Algorithms.cc:23-35; its harness is two-sided).  Side i holds the
    buffers of standalone kernel names[i]; launches are lists of (kernel, sides)."""

    def __init__(self, names: Sequence[str], device: int = 0):
        self.l = _lib.lib()
        _lib.check(self.l.bfuse_init(device))
        if not 2 <= len(names) <= _lib.MAXK:
            raise ValueError(f"a group has 2 .. {_lib.MAXK} kernels")
        self.k = [kernel_info(n) for n in names]
        self.live_sides = []
        try:
            for side, k in enumerate(self.k, 1):
                if k.kind != 0:
                    raise ValueError(f"{k.name} is a fused kernel; sides must be standalone kernels")
                _lib.check(self.l.bfuse_set_elem_bytes(side, *k.elem_bytes))
                _lib.check(self.l.bfuse_initialize_side(side, *[_i4(s) for s in k.shapes]))
                self.live_sides.append(side)
        except Exception:
            self.close()
            raise

    def close(self):
        while self.live_sides:
            _lib.check(self.l.bfuse_finalize_side(self.live_sides.pop()))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def fused(self, kind: str, suffix: str = "") -> KernelHandle:
        return kernel_info("_".join(k.name for k in self.k) + f"_fused_{kind}{suffix}")

    def set_plan(self, fused: KernelHandle, plan, workgroups: Optional[int] = None) -> KernelHandle:
        _lib.check(self.l.bfuse_set_plan(fused.func, C.byref(plan.c)))
        n = plan.fused_grid if workgroups is None else min(int(workgroups), plan.fused_grid)
        return replace(fused, grid=(n, 1, 1))

    def upload(self, side: int, I, F):
        k = self.k[side]
        a = [np.ascontiguousarray(x, dtype=_DT[k.elem_bytes[i]]) for i, x in enumerate((I, F))]
        for i in range(2):
            if a[i].size != int(np.prod(k.shapes[i])):
                raise ValueError(f"{k.name}: tensor {i} has {a[i].size} elements, kernel expects {int(np.prod(k.shapes[i]))}")
        _lib.check(self.l.bfuse_upload(side + 1, a[0].ctypes.data, a[1].ctypes.data))

    def zero_outputs(self):
        for side in self.live_sides:
            _lib.check(self.l.bfuse_zero_output(side))

    def download(self, side: int) -> np.ndarray:
        k = self.k[side]
        O = np.empty(tuple(k.shapes[2]), _DT[k.elem_bytes[2]])
        _lib.check(self.l.bfuse_download(side + 1, O.ctypes.data))
        return O

    def _descs(self, launches):
        """launches: [(KernelHandle, (side, ...)), ...] with 0-based sides; a standalone kernel takes one."""
        arr = (_lib.LaunchDescC * len(launches))()
        for d, (k, sides) in zip(arr, launches):
            d.func = k.func
            d.grid[:] = k.grid
            d.block[:] = k.block
            d.n_sides = len(sides)
            for i, sd in enumerate(sides):
                d.sides[i] = sd + 1
        return arr

    def unfused(self):
        return [(k, (i,)) for i, k in enumerate(self.k)]

    def launch(self, launches):
        arr = self._descs(launches)
        _lib.check(self.l.bfuse_launch_list(len(arr), arr))

    def synchronize(self):
        _lib.check(self.l.bfuse_synchronize())

    def time(self, launches, warmup: int = 3, reps: int = 30):
        """(mean GPU-side microseconds of each launch, wall-clock microseconds per round when queued)."""
        arr = self._descs(launches)
        each = np.zeros(len(arr), np.float32)
        queued = C.c_float()
        _lib.check(self.l.bfuse_time_list(len(arr), arr, warmup, reps, each.ctypes.data_as(C.POINTER(C.c_float)), C.byref(queued)))
        return each, queued.value


class GenericOperation:
    """Two to four sides with caller-given (I, F, O) shapes, for kernels that come from a code object
    (the front end's output) rather than from the library's registry."""

    def __init__(self, *shapes, device: int = 0):
        self.l = _lib.lib()
        _lib.check(self.l.bfuse_init(device))
        if not 2 <= len(shapes) <= _lib.MAXK:
            raise ValueError(f"2 .. {_lib.MAXK} sides")
        self.shapes = [[_i4(s) for s in sh] for sh in shapes]
        self.nelem = [[int(np.prod(s)) for s in sh] for sh in shapes]
        self.modules = []
        self.live_sides = []
        try:
            for side in range(1, len(shapes) + 1):
                _lib.check(self.l.bfuse_set_elem_bytes(side, 4, 4, 4))
                _lib.check(self.l.bfuse_initialize_side(side, *self.shapes[side - 1]))
                self.live_sides.append(side)
        except Exception:
            self.close()
            raise

    def close(self):
        for m in self.modules:
            self.l.bfuse_module_unload(m)
        self.modules = []
        while self.live_sides:
            _lib.check(self.l.bfuse_finalize_side(self.live_sides.pop()))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def load(self, path: str) -> int:
        mid = C.c_int(-1)
        _lib.check(self.l.bfuse_module_load(path.encode(), C.byref(mid)))
        self.modules.append(mid.value)
        return mid.value

    def upload(self, side: int, I, F):
        I, F = np.ascontiguousarray(I, np.float32), np.ascontiguousarray(F, np.float32)
        assert I.size == self.nelem[side][0] and F.size == self.nelem[side][1]
        _lib.check(self.l.bfuse_upload(side + 1, I.ctypes.data, F.ctypes.data))

    def zero_outputs(self):
        for side in self.live_sides:
            _lib.check(self.l.bfuse_zero_output(side))

    def download(self, side: int) -> np.ndarray:
        O = np.empty(self.nelem[side][2], np.float32)
        _lib.check(self.l.bfuse_download(side + 1, O.ctypes.data))
        return O

    def launch(self, module: int, name: str, grid, block, n_ptrs: int, side: int = 0) -> float:
        us = C.c_float()
        _lib.check(self.l.bfuse_module_launch(module, name.encode(), _u3(grid), _u3(block), n_ptrs, side + 1 if n_ptrs == 3 else 0,
                                              C.byref(us)))
        return us.value


# ---- synthetic inputs ---------------------------------------------------------------------
def fill_uniform(seed: int, n: int, lo: float, hi: float) -> np.ndarray:
    out = np.empty(n, np.float32)
    _lib.lib().bfuse_fill_uniform(seed, n, lo, hi, out.ctypes.data)
    return out


def fill_normal(seed: int, n: int, mean: float, std: float) -> np.ndarray:
    out = np.empty(n, np.float32)
    _lib.lib().bfuse_fill_normal(seed, n, mean, std, out.ctypes.data)
    return out


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    _lib.lib().bfuse_f32_to_bf16(x.size, x.ctypes.data, out.ctypes.data)
    return out


def bf16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    _lib.lib().bfuse_bf16_to_f32(x.size, x.ctypes.data, out.ctypes.data)
    return out


def load_kernels(path: str) -> None:
    """Adds the fused kernels of a module built by build_pairs to the registry (found by name from then on)."""
    _lib.check(_lib.lib().bfuse_load_kernels(os.fspath(path).encode()))


def checksum_of(chunk: np.ndarray) -> np.ndarray:
    """What Operation.checksum_output reports for a chunk with these contents (a whole number of 32-bit words)."""
    w = np.ascontiguousarray(chunk).ravel().view(np.uint32).astype(np.uint64)
    pos = (np.arange(w.size, dtype=np.uint64) % np.uint64(65521)) + np.uint64(1)
    with np.errstate(over="ignore"):
        return np.array([w.sum(dtype=np.uint64), (w * pos).sum(dtype=np.uint64)], np.uint64)


def check_matrix(o: np.ndarray, o_ans: np.ndarray, eps: float = 1e-3) -> int:
    """check_matrix of the reference (utils_cc.py:52-85): number of wrong elements."""
    o, a = np.ascontiguousarray(o, np.float32), np.ascontiguousarray(o_ans, np.float32)
    assert o.size == a.size
    return _lib.lib().bfuse_check_matrix(o.ctypes.data, a.ctypes.data, o.size, eps)


def probe_placement(workgroups: int, threads: int = 256, hold: int = 2000) -> dict:
    """Where the hardware puts consecutive workgroup ids: arrays of XCD, shader engine, CU and SIMD
    per workgroup, plus start ticks."""
    l = _lib.lib()
    _lib.check(l.bfuse_init(0))
    out = {k: np.zeros(workgroups, np.uint32) for k in ("xcc", "se", "cu", "simd")}
    out["start"] = np.zeros(workgroups, np.uint64)
    _lib.check(l.bfuse_probe_placement(workgroups, threads, hold, out["xcc"].ctypes.data, out["se"].ctypes.data,
                                       out["cu"].ctypes.data, out["simd"].ctypes.data, out["start"].ctypes.data))
    return out


def device_name() -> str:
    buf = C.create_string_buffer(256)
    cus, lds, wave = C.c_int(), C.c_int(), C.c_int()
    _lib.check(_lib.lib().bfuse_device_info(buf, 256, C.byref(cus), C.byref(lds), C.byref(wave)))
    return f"{buf.value.decode()} CUs={cus.value} wave={wave.value}"
