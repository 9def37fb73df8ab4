"""Pair-matrix driver: run every (kernel1, kernel2) of two fusion sets in every mode, keep the
GPU-side traces, and tabulate speed-ups.

Counterpart of the reference's suite scripts:

  * scripts/profile_test_suite.py:13-140 -- the command matrix over `benchmark T K1 K2` for the
    methods kernel1, kernel2, parallel, hfuse, bfuse, 3 warm-up + 30 timed launches, one GPU
    trace per command (there: nsys; here: rocprofv3 --kernel-trace, or the library's own
    dispatch timestamps when run in-process);
  * scripts/analyze_test_suite.py:103-161 -- per-trace statistics (warm-ups dropped; for two
    kernels on two streams the span from the first start to the later end);
  * scripts/analyze_test_suite.py:425-428 -- serial = kernel1 + kernel2, speed-up = serial / variant.

The suite description is the reference's `info.yaml`: `FusionSet: [{Set: [...]}, {Set: [...]}]`.
Set members are kernel names of the library's registry (the reference's `KernelInfo` block,
operator shapes for TVM, is accepted and ignored: shapes are compiled into the kernels).

    python -m bfuse_project_amd.suite info.yaml -o OUT            # run in-process, write traces + tables
    python -m bfuse_project_amd.suite info.yaml -o OUT --commands # only print the rocprofv3 command matrix
    python -m bfuse_project_amd.suite info.yaml -o OUT --analyze  # tables from traces already under OUT/exec
"""
import argparse
import csv
import json
import os
import sys
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import yaml

METHODS = ["kernel1", "kernel2", "parallel", "hfuse", "bfuse"]   # profile_test_suite.py:25
WARMUP_TRIALS = 3                                                  # profile_test_suite.py:10-11
TIMED_TRIALS = 30


# ---- suite description ------------------------------------------------------------------
def load_info(path: str) -> dict:
    with open(path) as f:
        info = yaml.safe_load(f)
    sets = info.get("FusionSet") if isinstance(info, dict) else None
    if not isinstance(sets, list) or len(sets) != 2:
        raise ValueError("Number of fusion sets are only 2.")          # profile_test_suite.py:19-21
    for s in sets:
        if not isinstance(s, dict) or not isinstance(s.get("Set"), list) or not s["Set"]:
            raise ValueError("every FusionSet entry needs a non-empty 'Set' list")
    return info


def suite_dir_of(info_path: str) -> str:
    """The suite directory of `<suite>/config/info.yaml` (where configure wrote it)."""
    return os.path.dirname(os.path.dirname(os.path.abspath(info_path)))


def set_names(info: dict) -> Tuple[List[str], List[str]]:
    return list(info["FusionSet"][0]["Set"]), list(info["FusionSet"][1]["Set"])


def combos(info: dict, triangular: bool = False) -> List[Tuple[int, int]]:
    """Index pairs to run.  The reference's two sets list the same operators twice and it walks
    the upper triangle (`for kidx2 in range(kidx1, kernel2_size)`); with distinct sets the full
    matrix is wanted, which is the default here."""
    a, b = set_names(info)
    return [(i, j) for i in range(len(a)) for j in range(i if triangular else 0, len(b))]


# ---- command matrix (profile_test_suite.py:13-140) ----------------------------------------------
def _ids(info: dict, info_path: Optional[str]):
    """How a command names its kernels: with the suite's info.yaml at hand by position in the two sets
    (`-i info.yaml T idx1 idx2`, the reference's form: its benchmark switches on those positions,
    macro_h.py:296-320), without it by kernel name."""
    a, b = set_names(info)
    if info_path:
        return ["-i", os.path.abspath(info_path)], (lambda i: str(i)), (lambda j: str(j))
    return [], (lambda i: a[i]), (lambda j: b[j])


def bfuse_suffix(k1: str, k2: str) -> List[str]:
    """`-x suffix` selecting the block-fused variant of (k1, k2) when the library holds several and none
    under the plain name: the one the footprint rule selects, else the first registered."""
    from . import tuner
    from .operation import kernel_info
    variants = [h for h in tuner.built_variants(k1, k2) if h.kind == 1]
    stem = f"{k1}_{k2}_fused_bfuse"
    if len(variants) <= 1 or any(h.name == stem for h in variants):
        return []
    a, b = kernel_info(k1), kernel_info(k2)
    pick = tuner.find_variant(a, b, {"kind": "bfuse", "pattern": "chunked", "p0": 256, "p1": 1}) or variants[0]
    return ["-x", pick.name[len(stem):]]


def valid_commands(info: dict, benchmark_path: str, triangular: bool = False, info_path: Optional[str] = None,
                   resident: bool = False) -> List[List[str]]:
    """`benchmark -v T K1 K2` for every method and pair (profile_test_suite.py:13-47); `resident`: with the driver's
    -r (operands written and outputs compared on the device, for operators of several GB)."""
    a, b = set_names(info)
    opts, k1, k2 = _ids(info, info_path)
    common = [os.path.abspath(benchmark_path), "-v"] + (["-r"] if resident else []) + opts
    out = []
    for idx, _ in enumerate(METHODS):
        if idx == 0:
            out += [common + [str(idx), k1(i), k2(0)] for i in range(len(a))]
        elif idx == 1:
            out += [common + [str(idx), k1(0), k2(j)] for j in range(len(b))]
        else:
            out += [common + (bfuse_suffix(a[i], b[j]) if idx == 4 else []) + [str(idx), k1(i), k2(j)] for i, j in combos(info, triangular)]
    return out


def exec_commands(info: dict, benchmark_path: str, exec_path: str, triangular: bool = False, info_path: Optional[str] = None,
                  resident: bool = False) -> List[List[str]]:
    """One rocprofv3 kernel-trace run per (method, k1, k2); the trace lands in
    `<exec_path>/<method index>_<i>_<j>_kernel_trace.csv` (the reference's file naming with the
    profiler's suffix)."""
    a, b = set_names(info)
    opts, k1, k2 = _ids(info, info_path)
    bench = os.path.abspath(benchmark_path)
    n = str(WARMUP_TRIALS + TIMED_TRIALS)

    def one(idx, i, j):
        return ["rocprofv3", "--kernel-trace", "--output-format", "csv", "-d", exec_path, "-o", f"{idx}_{i}_{j}", "--",
                bench, "-n", n] + (["-r"] if resident else []) + opts + (bfuse_suffix(a[i], b[j]) if idx == 4 else []) + [str(idx), k1(i), k2(j)]
    out = []
    for idx, _ in enumerate(METHODS):
        if idx == 0:
            out += [one(idx, i, 0) for i in range(len(a))]
        elif idx == 1:
            out += [one(idx, 0, j) for j in range(len(b))]
        else:
            out += [one(idx, i, j) for i, j in combos(info, triangular)]
    return out


# ---- traces ---------------------------------------------------------------------------------
def write_trace(path: str, rows: Sequence[dict]) -> None:
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=["Start", "Duration", "Name"])
        w.writeheader()
        for r in rows:
            w.writerow({"Start": r["Start"], "Duration": r["Duration"], "Name": r["Name"]})


def read_trace(path: str) -> List[dict]:
    """Rows {Name, Start, Duration} (ns) in start order, from this module's own trace files,
    from rocprofv3's `*_kernel_trace.csv` (Kernel_Name, Start_Timestamp, End_Timestamp), or from the
    reference's nsys export (`Start (ns)`, `Duration (ns)`, `Name`)."""
    out = []
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            if "Kernel_Name" in r:
                s, e = float(r["Start_Timestamp"]), float(r["End_Timestamp"])
                out.append({"Name": r["Kernel_Name"], "Start": s, "Duration": e - s})
            elif "Start (ns)" in r:
                if not r.get("Duration (ns)"):
                    continue
                out.append({"Name": r["Name"], "Start": float(r["Start (ns)"]), "Duration": float(r["Duration (ns)"])})
            else:
                out.append({"Name": r["Name"], "Start": float(r["Start"]), "Duration": float(r["Duration"])})
    out.sort(key=lambda r: r["Start"])
    return out


def _stats(v: Sequence[float]) -> Tuple[float, float, float, float]:
    if not len(v):
        raise ValueError("no timed launches in the trace")
    a = np.asarray(v, np.float64)
    return float(a.min()), float(a.max()), float(a.mean()), float(a.std())


def single_statistics(rows: Sequence[dict], kernel_name: str, warmup: int = WARMUP_TRIALS):
    """(min, max, mean, std) of the durations of `kernel_name`, first `warmup` launches dropped
    (analyze_test_suite.py:103-124)."""
    d = [r["Duration"] for r in rows if r["Name"] == kernel_name]
    return _stats(d[warmup:])


def parallel_statistics(rows: Sequence[dict], kernel_names: Sequence[str], warmup: int = WARMUP_TRIALS):
    """Two kernels per repetition: the repetition's time is the first one's duration if it ends
    last, else the span from its start to the second one's end (analyze_test_suite.py:126-161)."""
    if len(kernel_names) != 2:
        raise ValueError("Number of kernel_names must be 2.")
    sel = [r for r in rows if r["Name"] in kernel_names][warmup * 2:]
    res = []
    for first, second in zip(sel[0::2], sel[1::2]):
        if first["Start"] + first["Duration"] > second["Start"] + second["Duration"]:
            res.append(first["Duration"])
        else:
            res.append(second["Start"] - first["Start"] + second["Duration"])
    return _stats(res)


# ---- in-process run -------------------------------------------------------------------------
def fused_variants(k1: str, k2: str) -> Dict[str, list]:
    """Fused kernels the library holds for (k1, k2), by kind ('hfuse' / 'bfuse')."""
    from .operation import list_kernels
    out = {"hfuse": [], "bfuse": []}
    for h in list_kernels():
        if h.sides == (k1, k2):
            if h.kind == 2:
                out["hfuse"].append(h)
            elif h.kind == 1:
                out["bfuse"].append(h)
    return out


def _synthetic(handle, seed):
    """Seeded U(-0.5, 0.5) operands, as the reference's harness fills them (utils_cc.py:28-31)."""
    from .operation import fill_uniform, f32_to_bf16
    if handle.name.startswith("rmsnorm_rope_bf16"):
        # second operand is a byte blob (bf16 weight, fp32 cos and sin tables of 128-wide heads)
        from .workloads import pack_norm_rope_operand, rope_tables
        rows, d = handle.shapes[0][0], handle.shapes[0][1]
        cosv, sinv = rope_tables(rows, 128, 500000.0)
        return [f32_to_bf16(fill_uniform(seed, rows * d, -0.5, 0.5)),
                pack_norm_rope_operand(f32_to_bf16(fill_uniform(seed + 1, d, 0.5, 1.5)), cosv, sinv)]
    out = []
    for idx in (0, 1):
        n = int(np.prod(handle.shapes[idx]))
        eb = handle.elem_bytes[idx]
        v = fill_uniform(seed + idx, n if eb != 1 else (n + 3) // 4, -0.5, 0.5)
        out.append(v if eb == 4 else f32_to_bf16(v) if eb == 2 else v.view(np.uint8)[:n].copy())
    return out


def read_own(path: str, name: str) -> List[float]:
    """Durations (ns) of `name` in a trace, warm-ups dropped."""
    return [r["Duration"] for r in read_trace(path) if r["Name"] == name][WARMUP_TRIALS:]


def _fill_on_device(op, side: int, seed: int) -> bool:
    """The operands `_synthetic` would upload, written in HBM instead; False for a side with operands the
    device fill does not write (byte blobs)."""
    k = op.k[side]
    if k.name.startswith("rmsnorm_rope_bf16") or any(e not in (2, 4) for e in k.elem_bytes[:2]):
        return False
    op.fill_uniform_device(side, 0, seed, -0.5, 0.5)
    op.fill_uniform_device(side, 1, seed + 1, -0.5, 0.5)
    return True


def _chunks(handle) -> int:
    """Elements per checksum chunk of a kernel's output: the output cut into as many chunks (up to 1024) as divide it."""
    total = int(np.prod(handle.shapes[2]))
    unit = 4 // handle.elem_bytes[2] if handle.elem_bytes[2] < 4 else 1
    for n in (1024, 512, 256, 128, 64, 32, 16, 8, 4, 2, 1):
        if total % n == 0 and (total // n) % unit == 0:
            return total // n
    return total


def run_suite(info: dict, out_dir: str, validate: bool = True, triangular: bool = False, log=print, resident: bool = False,
              rows: Optional[Tuple[int, int]] = None) -> List[dict]:
    """Runs the matrix over resident buffers with the library's dispatch timestamps, writes one
    trace per (method, i, j) under `<out_dir>/exec/` and returns the analysed rows.

    `resident`: for operators whose operands and results run to GB (the reference's benchmark.yaml: every
    operator at batch 1024) -- the same uniform operands are written on the device instead of being filled on
    the host and copied, a fused kernel's outputs are compared with the unfused kernels' through checksums
    computed on the device (up to 1024 chunks per output) instead of being copied back, and long kernels are
    sampled fewer than 30 times (at least 5) so that a mode takes about a quarter of a second.
    `rows` = (lo, hi): only the pairs whose first operator is lo <= i < hi of the first set (a long matrix run in
    parts; the traces of all parts under one `exec/` are analysed together with --analyze)."""
    from . import tuner
    from .operation import Operation
    a, b = set_names(info)
    exec_dir = os.path.join(out_dir, "exec")
    os.makedirs(exec_dir, exist_ok=True)
    n_rep = TIMED_TRIALS

    def trace_of(t_tot, t_a, t_b, names):
        rows, clock = [], 0.0
        for r in range(len(t_tot)):
            if len(names) == 1:
                rows.append({"Name": names[0], "Start": clock, "Duration": float(t_tot[r]) * 1e3})
            else:
                # two dispatches: the first starts the repetition, the second ends it
                rows.append({"Name": names[0], "Start": clock, "Duration": float(t_a[r]) * 1e3})
                rows.append({"Name": names[1], "Start": clock + (float(t_tot[r]) - float(t_b[r])) * 1e3, "Duration": float(t_b[r]) * 1e3})
            clock += float(t_tot[r]) * 1e3 + 1e3
        return rows

    for i, j in combos(info, triangular):
        if rows is not None and not rows[0] <= i < rows[1]:
            continue
        k1, k2 = a[i], b[j]
        with Operation(k1, k2) as op:
            on_device = [False, False]
            for side, seed in ((0, 0xB5F05E + 2 * i), (1, 0xB5F05E + 1000 + 2 * j)):
                on_device[side] = resident and _fill_on_device(op, side, seed)
            I1, F1 = (None, None) if on_device[0] else _synthetic(op.k[0], 0xB5F05E + 2 * i)
            I2, F2 = (None, None) if on_device[1] else _synthetic(op.k[1], 0xB5F05E + 1000 + 2 * j)
            if not on_device[0]:
                op.upload(0, I1, F1)
            if not on_device[1]:
                op.upload(1, I2, F2)
            base = None
            if validate and resident:
                op.zero_outputs()
                op.launch("serial")
                base = (op.checksum_output(0, _chunks(op.k[0])), op.checksum_output(1, _chunks(op.k[1])))
                if not (base[0][:, 0].any() and base[1][:, 0].any()):
                    raise RuntimeError(f"{k1} / {k2}: an unfused kernel wrote nothing")
            elif validate:
                base = (op.run_kernel(0, I1, F1), op.run_kernel(1, I2, F2))
                op.upload(0, I1, F1)
                op.upload(1, I2, F2)
            if resident:
                est = float(np.mean(op.time("serial", warmup=1, reps=2)[0]))
                n_rep = int(min(TIMED_TRIALS, max(5, 0.25e6 / max(est, 1.0))))
            # warm-ups are part of the trace, as in the reference's -n 33 runs
            t = op.time("kernel1", warmup=0, reps=WARMUP_TRIALS + n_rep)
            write_trace(os.path.join(exec_dir, f"0_{i}_0.csv"), trace_of(t[0], t[1], t[2], [k1]))
            t = op.time("kernel2", warmup=0, reps=WARMUP_TRIALS + n_rep)
            write_trace(os.path.join(exec_dir, f"1_0_{j}.csv"), trace_of(t[0], t[1], t[2], [k2]))
            t = op.time("parallel", warmup=0, reps=WARMUP_TRIALS + n_rep)
            write_trace(os.path.join(exec_dir, f"2_{i}_{j}.csv"), trace_of(t[0], t[1], t[2], [k1, k2]))
            # The chooser decides BEFORE any fused kernel of the pair has run, from the two kernels' footprints
            # (registers, LDS, barriers, launch shapes: the code objects' metadata) and their standalone
            # times just measured (KernelInfo.ExecTime): thread-level fusion, block fusion, or leave the
            # pair unfused.  The fused variants are all timed below for the table; `chooser` names the one
            # form this suite would run.
            t1 = float(np.mean(read_own(os.path.join(exec_dir, f"0_{i}_0.csv"), k1)))
            t2 = float(np.mean(read_own(os.path.join(exec_dir, f"1_0_{j}.csv"), k2)))
            choice = tuner.static_plan(op.k[0], op.k[1], kinds=("hfuse", "bfuse", "none"), times=(t1 / 1e3, t2 / 1e3))
            picked = tuner.find_variant(op.k[0], op.k[1], choice)
            st = choice["static"]
            with open(os.path.join(exec_dir, f"choice_{i}_{j}.json"), "w") as f:
                json.dump({"kind": choice["kind"] if picked is not None or choice["kind"] == "none" else "none",
                           "kernel": picked.name if picked is not None else None,
                           "not_built": picked is None and choice["kind"] != "none",
                           "side_by_side": bool(st["side_by_side"]), "needed": list(st["needed"]),
                           "cap_lds": st["cap_lds"], "cap_waves": st["cap_waves"], "predicted_us": st["predicted_us"]}, f)
            for kind, idx in (("hfuse", 3), ("bfuse", 4)):
                best = None
                for h in fused_variants(k1, k2)[kind]:
                    if validate and resident:
                        op.zero_outputs()
                        op.launch(kind, h)
                        got = (op.checksum_output(0, _chunks(op.k[0])), op.checksum_output(1, _chunks(op.k[1])))
                        if not (np.array_equal(got[0], base[0]) and np.array_equal(got[1], base[1])):
                            raise RuntimeError(f"{h.name}: output differs from the unfused kernels")
                    elif validate:
                        op.zero_outputs()
                        Q1, Q2 = op.run_fuse(h, I1, F1, I2, F2)
                        if not (np.array_equal(Q1.view(np.uint8), base[0].view(np.uint8)) and np.array_equal(Q2.view(np.uint8), base[1].view(np.uint8))):
                            raise RuntimeError(f"{h.name}: output differs from the unfused kernels")
                    t = op.time(kind, h, warmup=0, reps=WARMUP_TRIALS + n_rep)
                    if picked is not None and h.name == picked.name:
                        write_trace(os.path.join(exec_dir, f"chosen_{i}_{j}.csv"), trace_of(t[0], t[1], t[2], [h.name]))
                    m = float(np.mean(t[0][WARMUP_TRIALS:]))
                    if best is None or m < best[0]:
                        best = (m, h, t)
                if best:
                    _, h, t = best
                    write_trace(os.path.join(exec_dir, f"{idx}_{i}_{j}.csv"), trace_of(t[0], t[1], t[2], [h.name]))
                    with open(os.path.join(exec_dir, f"{idx}_{i}_{j}.name"), "w") as f:
                        f.write(h.name + "\n")
        log(f"[suite] {k1} x {k2} done")
    return analyze(info, exec_dir, triangular)


# ---- tables (analyze_test_suite.py:425-428) -----------------------------------------------------
def _find(exec_dir: str, stem: str) -> Optional[str]:
    for suffix in (".csv", "_kernel_trace.csv"):
        p = os.path.join(exec_dir, stem + suffix)
        if os.path.exists(p):
            return p
    return None


def analyze(info: dict, exec_dir: str, triangular: bool = False) -> List[dict]:
    a, b = set_names(info)
    rows = []
    for i, j in combos(info, triangular):
        k1, k2 = a[i], b[j]
        p1, p2 = _find(exec_dir, f"0_{i}_0"), _find(exec_dir, f"1_0_{j}")
        if not p1 or not p2:
            continue
        t1 = single_statistics(read_trace(p1), k1)[2]
        t2 = single_statistics(read_trace(p2), k2)[2]
        row = {"kernel1": k1, "kernel2": k2, "kernel1_ns": t1, "kernel2_ns": t2, "serial_ns": t1 + t2}
        pp = _find(exec_dir, f"2_{i}_{j}")
        if pp:
            row["parallel_ns"] = parallel_statistics(read_trace(pp), [k1, k2])[2]
            row["parallel_speedup"] = row["serial_ns"] / row["parallel_ns"]
        for kind, idx in (("hfuse", 3), ("bfuse", 4)):
            pf = _find(exec_dir, f"{idx}_{i}_{j}")
            if not pf:
                continue
            tr = read_trace(pf)
            name_file = os.path.join(exec_dir, f"{idx}_{i}_{j}.name")
            if os.path.exists(name_file):
                name = open(name_file).read().strip()
            else:
                name = next((r["Name"] for r in tr if r["Name"].startswith(f"{k1}_{k2}_fused_{kind}")), None)
            if name is None:
                continue
            row[f"{kind}_kernel"] = name
            row[f"{kind}_ns"] = single_statistics(tr, name)[2]
            row[f"{kind}_speedup"] = row["serial_ns"] / row[f"{kind}_ns"]
        # what the chooser decided for the pair (written by run_suite before the fused kernels ran) and the
        # time of that one form: the chosen fused kernel's, or the serial time when the pair is left unfused
        cf = os.path.join(exec_dir, f"choice_{i}_{j}.json")
        if os.path.exists(cf):
            with open(cf) as f:
                ch = json.load(f)
            row["chooser"] = ch
            row["chooser_ns"] = row["serial_ns"]
            if ch["kind"] != "none" and ch["kernel"]:
                pf = _find(exec_dir, f"{3 if ch['kind'] == 'hfuse' else 4}_{i}_{j}")
                # the trace of a kind holds the fastest variant; the chooser's kernel is timed in its own file
                own = _find(exec_dir, f"chosen_{i}_{j}")
                src = own or pf
                if src:
                    d = [r["Duration"] for r in read_trace(src) if r["Name"] == ch["kernel"]][WARMUP_TRIALS:]
                    if d:
                        row["chooser_ns"] = float(np.mean(d))
            row["chooser_speedup"] = row["serial_ns"] / row["chooser_ns"]
        rows.append(row)
    return rows


def geomean(values: Sequence[float]) -> float:
    v = np.asarray([x for x in values if x and x > 0], np.float64)
    return float(np.exp(np.log(v).mean())) if len(v) else float("nan")


def to_markdown(rows: Sequence[dict]) -> str:
    head = "| kernel1 | kernel2 | k1 us | k2 us | serial us | parallel | hfuse | bfuse | chooser | bfuse kernel |\n|---|---|---|---|---|---|---|---|---|---|\n"
    body = ""
    def chooser(r):
        if "chooser" not in r:
            return "-"
        c = r["chooser"]
        what = "unfused" if c["kind"] == "none" else c["kind"]
        if c.get("not_built"):
            what += " (chosen form not built)"
        return f"{what}: {r['chooser_ns'] / 1e3:.2f} ({r['chooser_speedup']:.2f}x)"

    for r in rows:
        def f(k):
            return f"{r[k + '_ns'] / 1e3:.2f} ({r[k + '_speedup']:.2f}x)" if k + "_ns" in r else "-"
        body += (f"| {r['kernel1']} | {r['kernel2']} | {r['kernel1_ns'] / 1e3:.2f} | {r['kernel2_ns'] / 1e3:.2f} | {r['serial_ns'] / 1e3:.2f} | "
                 f"{f('parallel')} | {f('hfuse')} | {f('bfuse')} | {chooser(r)} | {r.get('bfuse_kernel', '-')} |\n")
    kinds = [k for k in ("parallel", "hfuse", "bfuse") if any(k + "_speedup" in r for r in rows)]
    tail = "\ngeomean speed-up over serial: " + ", ".join(
        f"{k} {geomean([r.get(k + '_speedup') for r in rows]):.3f}x" for k in kinds)
    # what the table is for: each pair run in the fastest of its measured forms (serial counts as 1)
    best = [max([1.0] + [r[k + "_speedup"] for k in ("hfuse", "bfuse") if k + "_speedup" in r]) for r in rows]
    tail += f"; best form per pair, picked after the fact: {geomean(best):.3f}x ({sum(1 for x in best if x > 1.0)} of {len(rows)} pairs fused)"
    ch = [r for r in rows if "chooser" in r]
    if ch:
        fusedn = sum(1 for r in ch if r["chooser"]["kind"] != "none")
        tail += (f"\nthe chooser's form per pair (decided from the footprints and the two standalone times, before any fused kernel of the pair "
                 f"ran): {geomean([r['chooser_speedup'] for r in ch]):.3f}x ({fusedn} of {len(ch)} pairs fused, {len(ch) - fusedn} left unfused; "
                 f"worst {min(r['chooser_speedup'] for r in ch):.2f}x)")
    return head + body + tail + "\n"


def speedup_statistics(rows: Sequence[dict]) -> Dict[str, dict]:
    """max, min, geometric mean and standard deviation of every form's speed-up over serial: the block the reference
    prints under its figure (scripts/analyze_test_suite.py:1203-1209), plus the chooser's form."""
    out = {}
    for k in ("parallel", "hfuse", "bfuse", "chooser"):
        v = [r[k + "_speedup"] for r in rows if k + "_speedup" in r]
        if v:
            out[k] = {"pairs": len(v), "max": float(np.max(v)), "min": float(np.min(v)), "avg": geomean(v), "std": float(np.std(v))}
    return out


def draw_speedup_figure(rows: Sequence[dict], path: str, per_row: int = 21) -> str:
    """The reference's speed-up figure (scripts/analyze_test_suite.py:1134-1201, its `exec_figure.png`): one group of bars
    per pair -- two streams, thread-level fusion, block fusion, and here also the chooser's form -- 21 pairs to a row of
    the figure, the serial baseline dashed at 1, the y axis 0 .. 2, and the geometric means after the last pair."""
    import math
    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt
    forms = [k for k in ("parallel", "hfuse", "bfuse", "chooser") if any(k + "_speedup" in r for r in rows)]
    n, width = len(rows), 0.8 / max(len(forms), 1)
    n_rows = max(1, math.ceil(n / per_row))
    fig, axes = plt.subplots(n_rows, 1, figsize=(10, 1.6 * n_rows + 0.6), squeeze=False)
    for a in range(n_rows):
        ax = axes[a][0]
        lo, hi = a * per_row, min(n, (a + 1) * per_row)
        x = np.arange(hi - lo)
        for f, k in enumerate(forms):
            ax.bar(x + (f - (len(forms) - 1) / 2) * width, [rows[i].get(k + "_speedup", 0.0) for i in range(lo, hi)], width=width, label=k)
        ax.axhline(y=1, color="r", linewidth=0.5, linestyle="--")
        ax.set_ylim(0, 2)
        ax.set_ylabel("Speed up", fontsize=6)
        ax.tick_params(axis="both", labelsize=5)
        ax.set_xticks(x)
        ax.set_xticklabels([str(i) for i in range(lo, hi)])
        if a == n_rows - 1:       # the geometric means, one slot to the right of the last pair
            ax.axvline(x=x[-1] + 1, color="gray", linewidth=0.5, linestyle="--")
            for f, k in enumerate(forms):
                ax.bar([x[-1] + 2 + (f - (len(forms) - 1) / 2) * width], [geomean([r.get(k + "_speedup") for r in rows])], width=width,
                       color=f"C{f}")
        if a == 0:
            ax.legend(ncol=len(forms), loc="upper left", fontsize=5)
    fig.tight_layout()
    fig.savefig(path, dpi=200)
    plt.close(fig)
    return path


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("file", help="info.yaml with the two fusion sets")
    ap.add_argument("-o", dest="out", default="suite_out", help="output directory")
    ap.add_argument("--commands", action="store_true", help="print the rocprofv3 command matrix and exit")
    ap.add_argument("--analyze", action="store_true", help="only analyse traces already under OUT/exec")
    ap.add_argument("--triangular", action="store_true", help="walk the upper triangle as the reference does")
    ap.add_argument("--no-validate", action="store_true")
    ap.add_argument("--rows", metavar="LO:HI", help="run only the pairs whose first operator is LO <= i < HI of the first set")
    ap.add_argument("--resident", action="store_true", help="operands written and results compared on the device (operators at batch 1024)")
    ap.add_argument("--figure", action="store_true", help="also draw OUT/exec_figure.png, the reference's speed-up figure, and print its statistics")
    ap.add_argument("--benchmark", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "benchmark"))
    args = ap.parse_args(argv)
    try:
        info = load_info(args.file)
    except (OSError, ValueError) as e:
        print(f"error: {e}", file=sys.stderr)
        return 1
    exec_dir = os.path.join(args.out, "exec")
    # fused kernels built for this suite after the library (build_pairs): this process loads them, the
    # driver's processes find them through the environment
    from . import build_pairs
    try:
        modules = build_pairs.load_suite_modules(suite_dir_of(args.file))
    except Exception as e:
        print(f"error: {e}", file=sys.stderr)
        return 1
    if args.commands:
        prefix = f"BFUSE_KERNEL_MODULES={':'.join(modules)} " if modules else ""
        for c in exec_commands(info, args.benchmark, exec_dir, args.triangular, args.file, resident=args.resident):
            print(prefix + " ".join(c))
        return 0
    rows = analyze(info, exec_dir, args.triangular) if args.analyze else run_suite(info, args.out, not args.no_validate, args.triangular, resident=args.resident,
                                                                                        rows=tuple(int(x) for x in args.rows.split(":")) if args.rows else None)
    os.makedirs(args.out, exist_ok=True)
    with open(os.path.join(args.out, "summary.json"), "w") as f:
        json.dump(rows, f, indent=1)
    md = to_markdown(rows)
    with open(os.path.join(args.out, "summary.md"), "w") as f:
        f.write(md)
    print(md)
    if args.figure:
        print("==== EXEC_FIGURE ====\n---------------------------------------")
        for k, st in speedup_statistics(rows).items():
            print(f"{k:8s} | max: {st['max']}, min: {st['min']}, avg: {st['avg']}, std: {st['std']}")
        print("---------------------------------------")
        print(draw_speedup_figure(rows, os.path.join(args.out, "exec_figure.png")))
    return 0


if __name__ == "__main__":
    sys.exit(main())
