"""Which CU runs which workgroup of a block-fused launch, and how the two operators mix on every CU.

The reference's hardware-scheduler experiment: a fused kernel prints `Block: b SM: s` from `%smid`
(horizontal-fuser/src/Matchers.cc:573-581) and tests/interleave_scheduler/test/test_scheduler.py:7-131 reads
that log -- per SM the blocks it received in ascending order, each classified by the fused kernel's own
`blockIdx` test (its `check()`), then the SM with the most and the least one-sided mix (`Max Diff.`,
`Min Diff.`) and the mean of |n0 - n1| / (n0 + n1) over the SMs (`Mean Diff.`), and a coloured map with one
column per SM and one row per arrival.

Here the placement comes from the library's probe (`bfuse_probe_placement`: every workgroup of a launch of the
fused kernel's shape records XCC_ID and HW_ID -- XCD, shader engine, CU -- and holds its slot), the side of
every workgroup id from the dispatch plan itself (`bfuse_map_block`, the map the fused kernel evaluates), and
the statistics are the reference's.  Besides the per-CU mix it reports the per-XCD mix: on MI355X consecutive
workgroup ids go to consecutive XCDs, so a 1:1 interleave of two operators puts each of them on four of the
eight XCDs (their L2s, their CUs) -- the reason the library interleaves in chunks of 256.

    python -m bfuse_project_amd.scheduler_probe [--pattern zigzag|proportional|chunked|ranges] [--p0 N] [--p1 N]
                                                [--grids G1 G2] [--threads T] [--first N] [--rows N] [--no-color]
"""
import argparse
import sys
from typing import Dict, Optional, Sequence

import numpy as np

RED, BLUE, RESET = "\033[31m", "\033[34m", "\033[0m"


def cu_index(xcc: np.ndarray, se: np.ndarray, cu: np.ndarray) -> np.ndarray:
    """One number per physical CU: the distinct (XCD, shader engine, CU) triples in ascending order, 0 .. n-1."""
    key = xcc.astype(np.int64) * 10000 + se.astype(np.int64) * 100 + cu.astype(np.int64)
    return np.unique(key, return_inverse=True)[1]


def mix_statistics(unit_of_block: Sequence[int], side_of_block: Sequence[int], first: Optional[int] = None) -> Dict:
    """The statistics of test_scheduler.py:77-112 over units (CUs, or XCDs): per unit the number of blocks of
    side 0 and side 1 among the first `first` workgroup ids; the unit with the largest and the smallest
    |n0 - n1| with its shares; the mean over the units of |n0 - n1| / (n0 + n1)."""
    unit = np.asarray(unit_of_block, np.int64)
    side = np.asarray(side_of_block, np.int64)
    if unit.shape != side.shape or unit.ndim != 1 or unit.size == 0:
        raise ValueError("one unit and one side per workgroup id")
    if first is not None:
        unit, side = unit[:first], side[:first]
    n_units = int(unit.max()) + 1
    n0 = np.bincount(unit[side == 0], minlength=n_units)
    n1 = np.bincount(unit[side == 1], minlength=n_units)
    used = (n0 + n1) > 0
    diff = np.abs(n0 - n1)
    rel = diff[used] / (n0 + n1)[used]
    ids = np.flatnonzero(used)
    hi, lo = ids[int(np.argmax(diff[used]))], ids[int(np.argmin(diff[used]))]
    share = lambda u: (float(n0[u] / (n0[u] + n1[u])), float(n1[u] / (n0[u] + n1[u])))
    return {"units": int(used.sum()), "n0": n0, "n1": n1, "max_unit": int(hi), "max_share": share(hi),
            "min_unit": int(lo), "min_share": share(lo), "mean_diff": float(rel.mean())}


def arrival_map(unit_of_block: Sequence[int], side_of_block: Sequence[int], rows: int = 70, first: Optional[int] = None,
                color: bool = True) -> str:
    """The map of test_scheduler.py:114-131: one column per unit, row r = the side (0 / 1) of the r-th workgroup
    id the unit received (ascending ids), blank where a unit received fewer."""
    unit = np.asarray(unit_of_block, np.int64)
    side = np.asarray(side_of_block, np.int64)
    if first is not None:
        unit, side = unit[:first], side[:first]
    n_units = int(unit.max()) + 1
    cols = [side[unit == u][:rows] for u in range(n_units)]
    out = []
    for r in range(min(rows, max(len(c) for c in cols))):
        line = []
        for c in cols:
            if r >= len(c):
                line.append(" ")
            elif color:
                line.append((RED if c[r] == 0 else BLUE) + str(int(c[r])) + RESET)
            else:
                line.append(str(int(c[r])))
        out.append("".join(line))
    return "\n".join(out)


def probe(pattern: str, grids: Sequence[int], threads: int = 256, p0: int = 1, p1: int = 1, hold: int = 2000) -> Dict:
    """Launches the placement probe in the shape of the fused kernel of two operators with `grids` workgroups
    and returns, per workgroup id, its side under the plan, its CU (0 .. n-1) and its XCD."""
    from .operation import probe_placement
    from .patterns import LaunchDims, plan_blocks
    if len(grids) != 2:
        raise ValueError("two operators")
    plan = plan_blocks(pattern, [LaunchDims((int(g), 1, 1), (threads, 1, 1)) for g in grids], p0, p1)
    side, _ = plan.table()
    p = probe_placement(plan.fused_grid, threads, hold)
    xcd = (p["xcc"].astype(np.int64) - int(p["xcc"][0])) % 8     # the XCD of id 0 depends on where the last dispatch stopped
    return {"side": side, "cu": cu_index(p["xcc"], p["se"], p["cu"]), "xcd": xcd, "fused_grid": plan.fused_grid}


def report(r: Dict, first: Optional[int] = None, rows: int = 0, color: bool = True) -> str:
    """The text test_scheduler.py prints (its `SMs:` line reads `CUs:` here), the same for the XCDs, then the map."""
    out = []
    for label, key in (("CUs", "cu"), ("XCDs", "xcd")):
        s = mix_statistics(r[key], r["side"], first)
        out.append(f"{label}:    0 ~ {int(np.max(r[key]))}")
        out.append(f"Max Diff.:  {abs(s['max_share'][0] - s['max_share'][1]):.2f} ({s['max_share'][0]:.2f} : {s['max_share'][1]:.2f})")
        out.append(f"Min Diff.:  {abs(s['min_share'][0] - s['min_share'][1]):.2f} ({s['min_share'][0]:.2f} : {s['min_share'][1]:.2f})")
        out.append(f"Mean Diff.: {s['mean_diff']:.2f}")
    if rows:
        out.append(arrival_map(r["cu"], r["side"], rows, first, color))
    return "\n".join(out)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="Per-CU and per-XCD mix of the two operators of a block-fused launch.")
    ap.add_argument("--pattern", choices=("zigzag", "proportional", "chunked", "ranges"), default="zigzag")
    ap.add_argument("--p0", type=int, default=1, help="first pattern parameter (zigzag: M; proportional: MinOption; chunked: workgroups per chunk)")
    ap.add_argument("--p1", type=int, default=1, help="second pattern parameter (zigzag: N)")
    ap.add_argument("--grids", type=int, nargs=2, default=(2048, 2048), metavar=("G1", "G2"), help="workgroups of the two operators")
    ap.add_argument("--threads", type=int, default=256)
    ap.add_argument("--first", type=int, default=None, help="only the first N workgroup ids (the reference reads 4000 lines of its log)")
    ap.add_argument("--rows", type=int, default=0, help="print the arrival map with this many rows (the reference prints 70)")
    ap.add_argument("--no-color", action="store_true")
    args = ap.parse_args(argv)
    try:
        r = probe(args.pattern, args.grids, args.threads, args.p0, args.p1)
    except Exception as e:
        print(f"scheduler_probe: {e}", file=sys.stderr)
        return 1
    print(f"{args.pattern} ({args.p0}, {args.p1}) over {args.grids[0]} + {args.grids[1]} workgroups of {args.threads} threads: {r['fused_grid']} ids")
    print(report(r, args.first, args.rows, not args.no_color))
    return 0


if __name__ == "__main__":
    sys.exit(main())
