"""Pattern / ratio chooser for a pair (or a group of up to four kernels), measured at run time.

The reference hard-codes the live pattern and its M, N in Contexts.cc:64-79 and sweeps ratios
by editing that file and rebuilding the tool and the suite for every point
(legacy/tests/single_bgemm_conv2d/auto.py:9-30: M in 1..512 with N = 1, then N in 1..512 with
M = 1).  Here the dispatch table of a `..._fused_bfuse_rt` kernel is data, so the same sweep is
a loop of `set_plan` + timed launches over resident buffers, and it also covers what the
reference never made selectable (its chunked and proportional patterns, plain ranges) and
persistent workgroups.

`static_choice` is the part that needs no measurement: it reads what the code objects say
(KernelInfo.Reg / LDS / HasBarriers, fields the reference parses and never uses) and prunes.
"""
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

from . import config, patterns
from .operation import KernelHandle, Operation


@dataclass
class Candidate:
    label: str
    pattern: str
    p0: int = 1
    p1: int = 1
    workgroups: Optional[int] = None   # None: one workgroup per fused block; else persistent


def ratio_sweep(max_ratio: int = 512) -> List[Candidate]:
    """The reference's sweep: M = 1, 2, 4, ... with N = 1, then N = 2, 4, ... with M = 1."""
    out = [Candidate("zigzag 1:1", "zigzag", 1, 1)]
    r = 2
    while r <= max_ratio:
        out.append(Candidate(f"zigzag M={r}", "zigzag", r, 1))
        out.append(Candidate(f"zigzag N={r}", "zigzag", 1, r))
        r *= 2
    return out


def default_candidates(g1: int, g2: int, cus: int = 256) -> List[Candidate]:
    small, big = min(g1, g2), max(g1, g2)
    out = [Candidate("ranges", "ranges")]
    for c in (cus // 4, cus // 2, cus, 2 * cus):
        if c < big:
            out.append(Candidate(f"chunk {c}", "chunked", c))
    out.append(Candidate("zigzag 1:1", "zigzag", 1, 1))
    r = 2
    while r <= max(2, big // max(small, 1)) and r <= 64:
        out.append(Candidate(f"zigzag M={r}", "zigzag", r, 1))
        r *= 2
    out.append(Candidate("proportional", "proportional", 1))
    for k in (1, 2, 4):
        if k * cus < g1 + g2:
            out.append(Candidate(f"chunk {cus}, {k * cus} persistent workgroups", "chunked", cus, 1, k * cus))
    return out


def static_choice(a: KernelHandle, b: KernelHandle, cus: int = 256, times: Optional[Sequence[float]] = None) -> dict:
    """What the code-object metadata alone says (no launch).  `times`: the two kernels' standalone
    durations in microseconds where they are known (KernelInfo.ExecTime, a field the reference
    parses and never uses): with them the rule also predicts whether block fusion pays."""
    ta, tb = (times if times is not None else (-1.0, -1.0))
    ka = config.KernelInfo(a.name, a.has_barriers, a.grid, a.block, max(a.regs, 1), float(ta))
    kb = config.KernelInfo(b.name, b.has_barriers, b.grid, b.block, max(b.regs, 1), float(tb))
    return config.choose_fusion(ka, kb, max(a.lds_bytes, 0), max(b.lds_bytes, 0), cus,
                                matrix=(getattr(a, "matrix", False), getattr(b, "matrix", False)))


def autotune(op: Operation, candidates: Optional[Sequence[Candidate]] = None, warmup: int = 20, reps: int = 100,
             cus: int = 256) -> List[dict]:
    """Times every candidate plan of the pair's run-time-plan kernel over the buffers `op` holds
    (upload operands first).  Returns rows sorted by mean GPU time; row 0 is the choice."""
    rt = op.fused_rt()
    dims = [k_.grid[0] for k_ in op.k]
    ldims = [patterns.LaunchDims(tuple(k_.grid), tuple(k_.block)) for k_ in op.k]
    rows = []
    for c in (candidates if candidates is not None else default_candidates(dims[0], dims[1], cus)):
        plan = patterns.plan_blocks(c.pattern, ldims, c.p0, c.p1)
        h = op.set_plan(rt, plan, c.workgroups)
        t = op.time("bfuse", h, warmup=warmup, reps=reps)[0]
        rows.append({"label": c.label, "pattern": c.pattern, "p0": c.p0, "p1": c.p1, "workgroups": h.grid[0],
                     "persistent": c.workgroups is not None,
                     "us_mean": float(np.mean(t)), "us_median": float(np.median(t)), "us_min": float(np.min(t)),
                     "us_std": float(np.std(t))})
    rows.sort(key=lambda r: r["us_mean"])
    return rows


_PATTERN_NAMES = {0: "zigzag", 1: "proportional", 2: "chunked", 3: "ranges"}


def _side_dims(k1: KernelHandle, k2: KernelHandle):
    return [patterns.LaunchDims(tuple(k1.grid), tuple(k1.block)), patterns.LaunchDims(tuple(k2.grid), tuple(k2.block))]


def built_variants(k1: str, k2: str) -> List[KernelHandle]:
    """Every compile-time fused kernel (block or thread fusion) the library holds for the sides (k1, k2)."""
    from .operation import list_kernels
    return [k for k in list_kernels() if k.kind in (1, 2) and k.sides == (k1, k2)]


def same_dispatch(plan_a, plan_b) -> bool:
    """Do two block plans send every fused block id to the same (kernel, block)?  Plans built from
    different patterns can coincide (chunk 256 over grids of at most 256 workgroups is plain ranges)."""
    if plan_a.fused_grid != plan_b.fused_grid:
        return False
    ka, va = plan_a.table()
    kb, vb = plan_b.table()
    return bool(np.array_equal(ka, kb) and np.array_equal(va, vb))


def static_plan(a: KernelHandle, b: KernelHandle, cus: int = 256, kinds: Sequence[str] = ("hfuse", "bfuse"),
                times: Optional[Sequence[float]] = None) -> dict:
    """The fusion the metadata alone selects, among the allowed kinds: thread-level fusion when the
    footprints allow it and the grids match, else block fusion in chunks of `chunk` workgroups
    (one chunk per round over the CUs).  With "none" among the kinds the answer may be to leave the
    pair unfused: when the footprint rule predicts that block fusion does not pay
    (config.choose_fusion) and thread-level fusion is not possible either.
    Returns {"kind", "pattern", "p0", "p1", "static"}."""
    st = static_choice(a, b, cus, times)
    if "none" in kinds and (st["fuse"] == "none" or st["fuse"] not in kinds):
        return {"kind": "none", "pattern": None, "p0": 0, "p1": 0, "static": st}
    if "none" in kinds and st["fuse"] == "hfuse":
        return {"kind": "hfuse", "pattern": None, "p0": 0, "p1": 0, "static": st}
    if "hfuse" in kinds and (st["prefer"] == "hfuse" or "bfuse" not in kinds):
        if not st["hfuse_ok"]:
            raise ValueError(f"{a.name} + {b.name}: thread-level fusion is not possible (barriers on both sides, threads or LDS)")
        return {"kind": "hfuse", "pattern": None, "p0": 0, "p1": 0, "static": st}
    return {"kind": "bfuse", "pattern": "chunked", "p0": int(st["chunk"]), "p1": 1, "static": st}


def find_variant(k1: KernelHandle, k2: KernelHandle, choice: dict) -> Optional[KernelHandle]:
    """The built compile-time kernel of (k1, k2) that realises `choice` (static_plan's or a row of
    autotune): for block fusion, the one whose dispatch table equals the chosen plan's."""
    if choice["kind"] == "none":
        return None
    built = built_variants(k1.name, k2.name)
    if choice["kind"] == "hfuse":
        hs = [k for k in built if k.kind == 2]
        return hs[0] if hs else None
    dims = _side_dims(k1, k2)
    want = patterns.plan_blocks(choice["pattern"], dims, max(choice["p0"], 1), max(choice["p1"], 1))
    for k in built:
        if k.kind != 1:
            continue
        have = patterns.plan_blocks(_PATTERN_NAMES[k.pattern], dims, max(k.p0, 1), max(k.p1, 1))
        if same_dispatch(want, have):
            return k
    return None


# ---- groups of more than two kernels (the fuser's Kernels list, Algorithms.cc:23-35) ---------------
def group_candidates(grids: Sequence[int], cus: int = 256) -> List[Candidate]:
    big = max(grids)
    out = [Candidate("ranges", "ranges")]
    for c in (cus // 4, cus // 2, cus, 2 * cus):
        if c < big:
            out.append(Candidate(f"chunk {c}", "chunked", c))
    out.append(Candidate("zigzag 1:1", "zigzag", 1, 1))
    out.append(Candidate("zigzag M=4", "zigzag", 4, 1))
    out.append(Candidate("proportional", "proportional", 1))
    for k in (1, 2, 4):
        if k * cus < sum(grids):
            out.append(Candidate(f"chunk {cus}, {k * cus} persistent workgroups", "chunked", cus, 1, k * cus))
    return out


def static_plan_group(kernels: Sequence[KernelHandle], cus: int = 256) -> dict:
    """The footprint rule for more than two kernels: block fusion in chunks of one round over the CUs
    (the largest LDS footprint is charged to every workgroup; `wg_per_cu` says how many then fit)."""
    lds = max(max(k.lds_bytes, 0) for k in kernels)
    regs = max(max(k.regs, 1) for k in kernels)
    fit = []
    for k in kernels:
        waves = -(-(k.block[0] * k.block[1] * k.block[2]) // 64)
        by_reg = (config.VGPRS_PER_SIMD // regs) * 4 // waves
        by_wave = config.MAX_WAVES_PER_SIMD * 4 // waves
        by_lds = config.LDS_PER_CU // lds if lds else 1 << 30
        fit.append(max(1, min(by_reg, by_wave, by_lds)))
    return {"kind": "bfuse", "pattern": "chunked", "p0": cus, "p1": 1, "static": {"wg_per_cu": tuple(fit), "chunk": cus}}


def built_group_variants(names: Sequence[str]) -> List[KernelHandle]:
    from .operation import list_kernels
    return [k for k in list_kernels() if k.kind in (1, 2) and k.sides == tuple(names)]


def find_group_variant(kernels: Sequence[KernelHandle], choice: dict) -> Optional[KernelHandle]:
    """The built compile-time kernel of the group whose dispatch table equals the chosen plan's."""
    dims = [patterns.LaunchDims(tuple(k.grid), tuple(k.block)) for k in kernels]
    want = patterns.plan_blocks(choice["pattern"], dims, max(choice["p0"], 1), max(choice["p1"], 1))
    for k in built_group_variants([k.name for k in kernels]):
        if k.kind == 1 and same_dispatch(want, patterns.plan_blocks(_PATTERN_NAMES[k.pattern], dims, max(k.p0, 1), max(k.p1, 1))):
            return k
    return None


def autotune_group(op, candidates: Optional[Sequence[Candidate]] = None, warmup: int = 20, reps: int = 100,
                   cus: int = 256) -> List[dict]:
    """autotune for a GroupOperation: times candidate plans on the group's run-time-plan kernel."""
    rt = op.fused("bfuse", "_rt")
    ldims = [patterns.LaunchDims(tuple(k.grid), tuple(k.block)) for k in op.k]
    sides = tuple(range(len(op.k)))
    rows = []
    for c in (candidates if candidates is not None else group_candidates([k.grid[0] for k in op.k], cus)):
        plan = patterns.plan_blocks(c.pattern, ldims, c.p0, c.p1)
        h = op.set_plan(rt, plan, c.workgroups)
        each, queued = op.time([(h, sides)], warmup=warmup, reps=reps)
        rows.append({"label": c.label, "pattern": c.pattern, "p0": c.p0, "p1": c.p1, "workgroups": h.grid[0],
                     "persistent": c.workgroups is not None, "us_mean": float(each[0]), "us_queued": float(queued)})
    rows.sort(key=lambda r: r["us_mean"])
    return rows
