#!/usr/bin/env python3
"""Writes the index-map golden vectors under tests/golden/ from files the reference holds.

Run in the build container only (the reference tree is not present on the GPU box):

    python tests/golden/make_pattern_goldens.py [/root/reference]

Everything is read as TEXT / YAML data; no reference code is imported or executed.
Inputs are *outputs of the reference's fuser* that the reference checked in:

  * config/kernels.yaml, bfuse_kernels.yaml, hfuse_kernels.yaml of the three generated
    suites (tests/benchmark, tests/inception_v3, tests/interleave_scheduler)
        -> fused_dims.json : unique (g1,t1,g2,t2) -> fused grid/block of both fusers.
  * the dispatch prologue (the `if / else if` chain over blockIdx.x) of emitted
    *_bfuse.cu / bfuse_kernels.cu files
        -> bfuse_maps.json : for sampled blockIdx values, the (KernelID_, NewBlockIdx_)
           that the emitted chain evaluates to.  The chain is evaluated by a small
           integer-expression evaluator over the emitted text, not by our oracle.
  * guards and `bar.sync` lines of emitted *_hfuse.cu / hfuse_kernels.cu files
        -> hfuse_ranges.json : thread range / block bound per side, barrier id+count.

  * config/*.yaml of legacy/tests/single_bgemm_conv2d/case-0_4/M_diff/case-2 (copied as is
    into config_sample/: they are the fuser's input/output data files).

Only numbers and config data are stored; no kernel body text is copied.
"""
import glob
import json
import os
import random
import re
import sys

import yaml

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.dirname(os.path.abspath(__file__))

_TOKEN_OK = re.compile(r"^[0-9b()\s+\-*/%<>=&|!]*$")


def _to_py(expr: str) -> str:
    """C integer expression over blockIdx.x -> Python expression over `b` (all operands are
    non-negative, so // and % agree with C)."""
    e = expr.replace("(int)blockIdx.x", "b").replace("int(", "(")
    e = e.replace("&&", " and ").replace("||", " or ")
    chk = e.replace("and", "&").replace("or", "|")
    if not _TOKEN_OK.match(chk):
        raise ValueError(f"unexpected token in emitted expression: {expr!r}")
    return re.sub(r"(?<![/])/(?![/])", "//", e)


def parse_bfuse_prologue(text: str):
    """Returns (kernel_names, branches, fused_threads); each branch is
    (cond_py, newblock_py, kernel_id, grid, block)."""
    head = text[: text.index("blockIdx_x_ = NewBlockIdx_")]
    names = re.findall(r"^\s*\*\s*(\d+): (\S+)\s*$", head, flags=re.M)
    names = [n for _, n in sorted((int(i), n) for i, n in names)]
    lb = re.search(r"__launch_bounds__\((\d+)\)", head)
    branches = []
    pat = re.compile(
        r"(?:else\s+)?if\s*(\(.*\))\s*\n\s*\{\s*\n\s*NewBlockIdx_ = (.*?);\s*\n\s*KernelID_\s*=\s*(\d+);"
        r"\s*\n\s*gridDim_x_ = (\d+);\s*\n\s*gridDim_y_ = (\d+);\s*\n\s*gridDim_z_ = (\d+);"
        r"\s*\n\s*blockDim_x_ = (\d+);\s*\n\s*blockDim_y_ = (\d+);\s*\n\s*blockDim_z_ = (\d+);"
    )
    for m in pat.finditer(head):
        cond, nb, kid, gx, gy, gz, bx, by, bz = m.groups()
        branches.append((_to_py(cond), _to_py(nb), int(kid), [int(gx), int(gy), int(gz)],
                         [int(bx), int(by), int(bz)]))
    return names, branches, int(lb.group(1))


def eval_chain(branches, b):
    for cond, nb, kid, grid, block in branches:
        if eval(cond, {"__builtins__": {}}, {"b": b}):
            return kid, eval(nb, {"__builtins__": {}}, {"b": b})
    return -1, -1


def sample_bids(total, bounds, rng, dense_limit=1200, n_random=120):
    if total <= dense_limit:
        return list(range(total))
    s = set()
    for c in list(bounds) + [0, total]:
        for d in range(-6, 7):
            if 0 <= c + d < total:
                s.add(c + d)
    for _ in range(n_random):
        s.add(rng.randrange(total))
    return sorted(s)


def bfuse_record(path, pattern, params, rng):
    text = open(path, errors="replace").read()
    names, branches, threads = parse_bfuse_prologue(text)
    kinfo = {}
    for _, _, kid, grid, block in branches:
        kinfo[kid] = (grid, block)
    n = len(names)
    grids = [kinfo[k][0] for k in range(n)]
    blocks = [kinfo[k][1] for k in range(n)]
    total = sum(g[0] * g[1] * g[2] for g in grids)
    bounds = set(int(x) for c, _, _, _, _ in branches for x in re.findall(r"\d+", c))
    samples = []
    for b in sample_bids(total, bounds, rng):
        k, v = eval_chain(branches, b)
        samples.append([b, k, v])
    # one id past the end must match no branch
    assert eval_chain(branches, total) == (-1, -1), path
    return {
        "source": os.path.relpath(path, REF),
        "pattern": pattern,
        "params": params,
        "grids": grids,
        "blocks": blocks,
        "fused_grid": total,
        "fused_block": threads,
        "samples": samples,
    }


def make_bfuse_maps():
    rng = random.Random(20240607)
    recs = []
    # (1) live 1:1 zig-zag, newest suite: a spread of pairs with distinct grid pairs
    files = sorted(glob.glob(f"{REF}/tests/benchmark/cuda/*_bfuse.cu"))
    seen = set()
    picked = []
    for f in files:
        txt = open(f, errors="replace").read(6000)
        g = tuple(re.findall(r"gridDim_[xyz]_ = (\d+);", txt)[:6])
        if g in seen:
            continue
        seen.add(g)
        picked.append(f)
    rng2 = random.Random(7)
    rng2.shuffle(picked)
    for f in sorted(picked[:40]):
        recs.append(bfuse_record(f, "zigzag", {"M": 1, "N": 1}, rng))
    # (2) ratio sweeps (M or N edited by sed in the reference's auto.py; the case directory
    #     name is the swept value, the other knob is 1)
    for f in sorted(glob.glob(f"{REF}/legacy/tests/single_bgemm_conv2d/case-*/*_diff/case-*/cuda/bfuse_kernels.cu")):
        m = re.search(r"/(M|N)_diff/case-(\d+)/", f)
        which, val = m.group(1), int(m.group(2))
        params = {"M": val, "N": 1} if which == "M" else {"M": 1, "N": val}
        recs.append(bfuse_record(f, "zigzag", params, rng))
    # (3) the only emitted SM-chunk prologue (TotalSM = 84)
    f = f"{REF}/legacy/tests/block_scheduler_test/cuda/bfuse_kernels.cu"
    recs.append(bfuse_record(f, "chunk", {"TotalSM": 84}, rng))
    json.dump(recs, open(f"{OUT}/bfuse_maps.json", "w"), separators=(",", ":"))
    print("bfuse_maps.json:", len(recs), "prologues,", sum(len(r["samples"]) for r in recs), "samples")


def make_hfuse_ranges():
    recs = []
    files = sorted(glob.glob(f"{REF}/legacy/tests/single_bgemm_conv2d/case-*/M_diff/case-1/cuda/hfuse_kernels.cu"))
    files += [f"{REF}/legacy/tests/block_scheduler_test/cuda/hfuse_kernels.cu"]
    files += sorted(glob.glob(f"{REF}/tests/benchmark/cuda/dense1_0_*_hfuse.cu"))[:12]
    guard = re.compile(
        r"if \(\(\(int\)threadIdx\.x >= (\d+) && \(int\)threadIdx\.x < (\d+)\) && "
        r"\(\(int\)blockIdx\.x >= 0 && \(int\)blockIdx\.x < (\d+)\)\)")
    for f in files:
        if not os.path.exists(f):
            continue
        text = open(f, errors="replace").read()
        lb = int(re.search(r"__launch_bounds__\((\d+)\)", text).group(1))
        sides = []
        for m in guard.finditer(text):
            seg = text[m.end(): m.end() + 1200]
            g = [int(x) for x in re.findall(r"\(int\)blockIdx\.x(?: /| %) ?(\d+)", seg)[:4]]
            decl = re.search(
                r"blockIdx_x_ = \(int\)blockIdx\.x % (\d+);\s*\n\s*int blockIdx_y_ = \(int\)blockIdx\.x / (\d+) % (\d+);"
                r"\s*\n\s*int blockIdx_z_ = \(int\)blockIdx\.x / (\d+);\s*\n\s*int threadIdx_x_ = \(\(int\)threadIdx\.x - (\d+)\) % (\d+);"
                r"\s*\n\s*int threadIdx_y_ = \(\(int\)threadIdx\.x - \d+\) / \d+ % (\d+);"
                r"\s*\n\s*int threadIdx_z_ = \(\(int\)threadIdx\.x - \d+\) / (\d+);", seg)
            gx, gx2, gy, gxy, off, bx, by, bxy = (int(v) for v in decl.groups())
            assert gx == gx2 and off == int(m.group(1))
            sides.append({"thr_lo": int(m.group(1)), "thr_hi": int(m.group(2)), "blocks": int(m.group(3)),
                          "grid_xy": [gx, gy, gxy], "block_xy": [bx, by, bxy]})
        bars = sorted(set((int(a), int(b)) for a, b in re.findall(r"bar\.sync (\d+), (\d+);", text)))
        recs.append({"source": os.path.relpath(f, REF), "fused_block": lb, "sides": sides,
                     "barriers": [list(b) for b in bars]})
    json.dump(recs, open(f"{OUT}/hfuse_ranges.json", "w"), separators=(",", ":"))
    print("hfuse_ranges.json:", len(recs), "files")


def make_fused_dims():
    rows = {}
    n_rows = 0
    suites = ["tests/benchmark", "tests/inception_v3", "tests/interleave_scheduler"]
    suites += [os.path.relpath(os.path.dirname(os.path.dirname(p)), REF) for p in
               sorted(glob.glob(f"{REF}/legacy/tests/single_bgemm_conv2d/case-0_4/M_diff/case-*/config/kernels.yaml"))]
    for s in suites:
        cfg = f"{REF}/{s}/config"
        kernels = yaml.safe_load(open(f"{cfg}/kernels.yaml"))
        fusions = yaml.safe_load(open(f"{cfg}/fusions.yaml"))
        bf = yaml.safe_load(open(f"{cfg}/bfuse_kernels.yaml"))
        hf = yaml.safe_load(open(f"{cfg}/hfuse_kernels.yaml"))

        def dims(e):
            return [e["GridDim"]["X"], e["GridDim"]["Y"], e["GridDim"]["Z"]], \
                   [e["BlockDim"]["X"], e["BlockDim"]["Y"], e["BlockDim"]["Z"]]

        for fu in fusions:
            k1, k2 = fu["Kernels"]
            g1, t1 = dims(kernels[k1])
            g2, t2 = dims(kernels[k2])
            b = bf[f"{k1}_{k2}_fused_bfuse"]
            h = hf[f"{k1}_{k2}_fused_hfuse"]
            n_rows += 1
            key = json.dumps([g1, t1, g2, t2])
            val = [*dims(b), *dims(h)]
            assert rows.get(key, val) == val
            rows[key] = val
    out = [{"k": json.loads(k), "bfuse": v[:2], "hfuse": v[2:]} for k, v in sorted(rows.items())]
    json.dump({"rows_read": n_rows, "unique": out}, open(f"{OUT}/fused_dims.json", "w"), separators=(",", ":"))
    print("fused_dims.json:", n_rows, "rows read,", len(out), "unique")


def copy_config_sample():
    """The four small YAML configs of one legacy case (two kernels, 152-thread conv block): data
    files in the fuser's wire format, one written by PyYAML and two by llvm::yaml."""
    import shutil
    src = f"{REF}/legacy/tests/single_bgemm_conv2d/case-0_4/M_diff/case-2/config"
    dst = f"{OUT}/config_sample"
    os.makedirs(dst, exist_ok=True)
    for n in ("kernels.yaml", "fusions.yaml", "bfuse_kernels.yaml", "hfuse_kernels.yaml"):
        shutil.copyfile(f"{src}/{n}", f"{dst}/{n}")
    print("config_sample/: 4 yaml files")


if __name__ == "__main__":
    copy_config_sample()
    make_fused_dims()
    make_bfuse_maps()
    make_hfuse_ranges()
