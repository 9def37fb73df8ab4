"""Fused kernels for the pairs of a configured suite that the library holds none for.

The reference generates a kernel per operator id with TVM, runs its fuser over EVERY pair of the two fusion
sets and compiles the result into the suite (scripts/configure_kernels.py:229-320, scripts/quick_start.py:44-55:
both fused forms per pair).  Here the operators are registered templates, so a fused kernel of any two of them is
one more instantiation: this module writes, for every pair of `<suite>/config/info.yaml` without a fused kernel,

    BFUSE_BFUSE_KERNEL(k1, <type of k1>, k2, <type of k2>, _c256, bfuse::kChunked, 256, 1)    block fusion
    BFUSE_HFUSE_KERNEL(k1, <type of k1>, k2, <type of k2>)                                    thread-level fusion
    BFUSE_BFUSE_RT_KERNEL(k1, <type of k1>, k2, <type of k2>)                                 block fusion, plan at run time (--rt)

into `<suite>/hip/pairs_<n>.hip` -- the operator types exactly as the library spells them
(bfuse_kernel_op_type) -- and builds `<suite>/hip/libbfuse_pairs.so` with the library's own flags and build
checks (csrc/Makefile, target `module`).  `<suite>/config/modules.yaml` then names the module; `suite`,
`quick_start` and `benchmark` (through BFUSE_KERNEL_MODULES) load it and find the new kernels by name.

    python -m bfuse_project_amd.build_pairs SUITE [--forms both|bfuse|hfuse] [--rt] [--chunk N] [--triangular] [--only K1+K2 ...] [-j J]

Thread-level fusion is written only where it can work: both workgroups fit one (at most 1024 threads and
160 KB of LDS together) and at most one side synchronises (config.choose_fusion's rule).
"""
import argparse
import os
import subprocess
import sys
from typing import Dict, List, Optional, Sequence, Tuple

import yaml

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LDS_PER_WORKGROUP = 160 * 1024
HEADERS = ("fuse.h", "ops_conv.h", "ops_conv_1x1.h", "ops_conv_general.h", "ops_conv_rect.h", "ops_gemm_bf16.h", "ops_gemm_f32.h", "ops_gemm_f32_dma.h",
           "ops_layout.h", "ops_pool.h", "ops_rowwise.h")


def op_type(name: str) -> str:
    from . import _lib
    t = _lib.lib().bfuse_kernel_op_type(name.encode())
    if not t:
        raise LookupError(f"{name}: not a standalone kernel of the library")
    return t.decode()


def op_lds(name: str) -> int:
    from . import _lib
    return int(_lib.lib().bfuse_kernel_op_lds(name.encode()))


def hfuse_possible(a, b, lds_a: int, lds_b: int) -> bool:
    """Can the two workgroups share one?  (threads, LDS, and at most one side with barriers)"""
    ta, tb = (int(k.block[0] * k.block[1] * k.block[2]) for k in (a, b))
    waves = -(-ta // 64) + -(-tb // 64)
    return waves * 64 <= 1024 and lds_a + lds_b + 16 <= LDS_PER_WORKGROUP and not (a.has_barriers and b.has_barriers)


def wanted(pairs: Sequence[Tuple[str, str]], registry: Dict[str, object], forms: str = "both", chunk: int = 256,
           lds=op_lds, rt: bool = False) -> List[dict]:
    """The fused kernels to build: [{k1, k2, form, name}], skipping what the registry already holds.
    `rt`: also the block-fused kernel whose dispatch plan is run-time data (`..._fused_bfuse_rt`), which the tuner
    times candidate plans and persistent workgroup counts on."""
    out, seen = [], set()
    for k1, k2 in pairs:
        for k in (k1, k2):
            if k not in registry or registry[k].kind != 0:
                raise LookupError(f"{k}: not a standalone kernel of the library")
        if (k1, k2) in seen:
            continue
        seen.add((k1, k2))
        if forms in ("both", "bfuse"):
            name = f"{k1}_{k2}_fused_bfuse_c{chunk}"
            if name not in registry:
                out.append({"k1": k1, "k2": k2, "form": "bfuse", "name": name})
        if rt:
            name = f"{k1}_{k2}_fused_bfuse_rt"
            if name not in registry:
                out.append({"k1": k1, "k2": k2, "form": "rt", "name": name})
        if forms in ("both", "hfuse") and hfuse_possible(registry[k1], registry[k2], lds(k1), lds(k2)):
            name = f"{k1}_{k2}_fused_hfuse"
            if name not in registry:
                out.append({"k1": k1, "k2": k2, "form": "hfuse", "name": name})
    return out


def source_text(kernels: Sequence[dict], chunk: int = 256, types=op_type) -> str:
    """One translation unit for `kernels` (entries of `wanted`)."""
    sides: Dict[str, str] = {}
    for k in kernels:
        for s in (k["k1"], k["k2"]):
            sides.setdefault(s, f"Side{len(sides)}")
    lines = ["// Written by bfuse_project_amd.build_pairs: fused kernels of registered operators for one suite."]
    lines += [f'#include "{h}"' for h in HEADERS]
    lines += ["", "using namespace bfuse;", "", "BFUSE_MODULE_PROLOGUE()", ""]
    lines += [f"using {alias} = {types(name)};   // {name}" for name, alias in sides.items()]
    lines.append("")
    for k in kernels:
        a, b = sides[k["k1"]], sides[k["k2"]]
        if k["form"] == "bfuse":
            lines.append(f"BFUSE_BFUSE_KERNEL({k['k1']}, {a}, {k['k2']}, {b}, _c{chunk}, bfuse::kChunked, {chunk}, 1)")
        elif k["form"] == "rt":
            lines.append(f"BFUSE_BFUSE_RT_KERNEL({k['k1']}, {a}, {k['k2']}, {b})")
        else:
            lines.append(f"BFUSE_HFUSE_KERNEL({k['k1']}, {a}, {k['k2']}, {b})")
    return "\n".join(lines) + "\n"


def spilling_kernels(res_text: str) -> List[str]:
    """Kernels a compilation's resource remarks report scratch memory or register spills for."""
    out, name = [], None
    for line in res_text.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:", 1)[1].split()[0]
        elif name and any(f"{what}: " in line and int(line.split(f"{what}: ", 1)[1].split()[0]) > 0
                          for what in ("ScratchSize [bytes/lane]", "VGPRs Spill", "SGPRs Spill")):
            if name not in out:
                out.append(name)
    return out


def _unit_kernel(line: str) -> Optional[str]:
    """The fused kernel a line of a written translation unit defines (or records as not built)."""
    if line.startswith("BFUSE_BFUSE_KERNEL("):
        a = [x.strip() for x in line[len("BFUSE_BFUSE_KERNEL("):-1].split(",")]
        return f"{a[0]}_{a[2]}_fused_bfuse{a[4]}"
    if line.startswith("BFUSE_BFUSE_RT_KERNEL("):
        a = [x.strip() for x in line[len("BFUSE_BFUSE_RT_KERNEL("):-1].split(",")]
        return f"{a[0]}_{a[2]}_fused_bfuse_rt"
    if line.startswith("BFUSE_HFUSE_KERNEL("):
        a = [x.strip() for x in line[len("BFUSE_HFUSE_KERNEL("):-1].split(",")]
        return f"{a[0]}_{a[2]}_fused_hfuse"
    if line.startswith("// not built"):
        return line.rsplit(": ", 1)[1].strip()
    return None


def written(hip_dir: str) -> List[str]:
    """Fused kernels the translation units of a suite already hold (built, to be built, or found not to fit)."""
    out = []
    if os.path.isdir(hip_dir):
        for f in sorted(os.listdir(hip_dir)):
            if f.startswith("pairs_") and f.endswith(".hip"):
                with open(os.path.join(hip_dir, f)) as fh:
                    out += [n for n in map(_unit_kernel, fh.read().splitlines()) if n]
    return out


def stale_units(hip_dir: str, types=None) -> List[str]:
    """Translation units that name a side by another type than the library gives that kernel now (the library was
    rebuilt with another tiling of the operator since they were written)."""
    types = types or op_type
    out = []
    if os.path.isdir(hip_dir):
        for f in sorted(os.listdir(hip_dir)):
            if f.startswith("pairs_") and f.endswith(".hip"):
                with open(os.path.join(hip_dir, f)) as fh:
                    for line in fh:
                        if line.startswith("using Side") and ";   // " in line:
                            typ = line.split(" = ", 1)[1].split(";   // ")[0]
                            name = line.rsplit("// ", 1)[1].strip()
                            try:
                                if types(name) != typ:
                                    out.append(f)
                                    break
                            except LookupError:
                                out.append(f)
                                break
    return out


def drop_spilling(hip_dir: str) -> List[str]:
    """Removes, from every pairs_*.hip whose last compilation reported spills, the kernels that spilled."""
    dropped = []
    for f in sorted(os.listdir(hip_dir)):
        if not (f.startswith("pairs_") and f.endswith(".res")):
            continue
        with open(os.path.join(hip_dir, f)) as fh:
            bad = spilling_kernels(fh.read())
        if not bad:
            continue
        src = os.path.join(hip_dir, f[:-4] + ".hip")
        with open(src) as fh:
            lines = fh.read().splitlines()
        keep = []
        for line in lines:
            name = None if line.startswith("//") else _unit_kernel(line)
            if name in bad:
                dropped.append(name)
                keep.append(f"// not built (does not fit the register file in this form): {name}")
            else:
                keep.append(line)
        with open(src, "w") as fh:
            fh.write("\n".join(keep) + "\n")
    return dropped


def suite_pairs(suite: str, triangular: bool = False) -> List[Tuple[str, str]]:
    """The suite's pairs of registry names; `triangular`: the upper triangle the reference profiles when its two
    sets list the same operators (scripts/profile_test_suite.py:13-47)."""
    with open(os.path.join(suite, "config", "info.yaml")) as f:
        info = yaml.safe_load(f)
    s0, s1 = (s["Set"] for s in info["FusionSet"])
    return [(s0[i], s1[j]) for i in range(len(s0)) for j in range(i if triangular else 0, len(s1))]


def module_paths(suite: str) -> List[str]:
    """The kernel modules a configured suite names (config/modules.yaml), as absolute paths."""
    p = os.path.join(suite, "config", "modules.yaml")
    if not os.path.exists(p):
        return []
    with open(p) as f:
        names = yaml.safe_load(f) or []
    return [n if os.path.isabs(n) else os.path.normpath(os.path.join(suite, n)) for n in names]


def load_suite_modules(suite: str) -> List[str]:
    """Loads the suite's modules into this process and returns their paths (for BFUSE_KERNEL_MODULES of children)."""
    from . import _lib
    paths = module_paths(suite)
    for p in paths:
        _lib.check(_lib.lib().bfuse_load_kernels(p.encode()))
    return paths


def build(suite: str, forms: str = "both", chunk: int = 256, only: Optional[Sequence[str]] = None, per_file: int = 2,
          jobs: int = 8, compile_: bool = True, triangular: bool = False, rt: bool = False) -> dict:
    """Writes <suite>/hip/pairs_*.hip for the suite's pairs that lack a fused kernel and builds the module.
    Returns {"kernels": [...], "files": [...], "module": path or None}."""
    from . import build_operators
    from .operation import list_kernels
    # the library's own kernels and the operators built for this suite's config (configure --build-missing: their
    # module is brought up to date and loaded); what an earlier run wrote for this suite is read from its
    # translation units below (the module of fused kernels is not loaded here: one built against older headers
    # would be refused, and is about to be rebuilt)
    build_operators.rebuild_and_load(suite, jobs)
    registry = {k.name: k for k in list_kernels()}
    pairs = suite_pairs(suite, triangular)
    if only:
        keep = {tuple(o.split("+", 1)) for o in only}
        unknown = keep - set(pairs)
        if unknown:
            raise LookupError(f"not pairs of this suite: {sorted(unknown)}")
        pairs = [p for p in pairs if p in keep]
    hip = os.path.join(suite, "hip")
    if stale_units(hip):
        # the library's operators changed under the suite's units: everything written for it is written again
        for f in os.listdir(hip):
            if f.startswith("pairs_") or f == "libbfuse_pairs.so":
                os.remove(os.path.join(hip, f))
    have = set(written(hip))       # units of an earlier, possibly interrupted, run are not written twice
    todo = [k for k in wanted(pairs, registry, forms, chunk, rt=rt) if k["name"] not in have]
    os.makedirs(hip, exist_ok=True)
    first = len([f for f in os.listdir(hip) if f.startswith("pairs_") and f.endswith(".hip")])
    files = []
    for i in range(0, len(todo), per_file):
        path = os.path.join(hip, f"pairs_{first + i // per_file}.hip")
        with open(path, "w") as f:
            f.write(source_text(todo[i:i + per_file], chunk))
        files.append(path)
    module = os.path.join(hip, "libbfuse_pairs.so")
    if not todo and not have:
        return {"kernels": [], "files": [], "module": None, "dropped": []}
    dropped: List[str] = []
    if compile_:      # make decides what is out of date (new units, or headers of the library that changed)
        cmd = ["make", "-C", CSRC, f"MODDIR={os.path.abspath(hip)}", f"-j{jobs}", "-k", "module"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            # A fused kernel that needs more registers than its launch bounds leave (a side that already fills the
            # register file, thread-fused with another) fails the library's no-spill check: such kernels are taken
            # out of their translation units and the build is run once more; anything else is an error.
            dropped = drop_spilling(hip)
            if not dropped:
                raise RuntimeError(f"building {module} failed:\n{r.stdout[-3000:]}\n{r.stderr[-3000:]}")
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"building {module} failed:\n{r.stdout[-3000:]}\n{r.stderr[-3000:]}")
            todo = [k for k in todo if k["name"] not in dropped]
        build_operators.name_module(suite, os.path.join("hip", "libbfuse_pairs.so"))
    return {"kernels": todo, "files": files, "module": module if compile_ else None, "dropped": dropped}


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="Build the fused kernels a configured suite lacks.")
    ap.add_argument("suite", help="directory written by bfuse_project_amd.configure")
    ap.add_argument("--forms", choices=("both", "bfuse", "hfuse"), default="both")
    ap.add_argument("--chunk", type=int, default=256, help="workgroups of one side per chunk of the block-fused dispatch (one round over the CUs)")
    ap.add_argument("--only", nargs="*", metavar="K1+K2", help="registry names of the pairs to build (default: every pair of the suite)")
    ap.add_argument("--triangular", action="store_true", help="only the pairs (i, j >= i) of two sets that list the same operators, as the reference profiles them")
    ap.add_argument("--rt", action="store_true", help="also the block-fused kernel with its dispatch plan as run-time data (for tuner.autotune and persistent workgroups)")
    ap.add_argument("--per-file", type=int, default=2, help="fused kernels per translation unit")
    ap.add_argument("-j", type=int, default=8, dest="jobs")
    ap.add_argument("--write-only", action="store_true", help="write the .hip files, do not compile")
    args = ap.parse_args(argv)
    try:
        r = build(args.suite, args.forms, args.chunk, args.only, args.per_file, args.jobs, not args.write_only, args.triangular, args.rt)
    except (LookupError, RuntimeError, OSError) as e:
        print(f"build_pairs: {e}", file=sys.stderr)
        return 1
    for k in r["kernels"]:
        print(k["name"])
    for name in r["dropped"]:
        print(f"not built (registers): {name}", file=sys.stderr)
    print(f"{len(r['kernels'])} fused kernels in {len(r['files'])} files" + (f"; module {r['module']}" if r["module"] else ""))
    return 0


if __name__ == "__main__":
    sys.exit(main())
