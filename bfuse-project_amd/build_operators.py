"""Operator kernels for the ids of a user config that no kernel of the library implements.

The reference generates one kernel per operator id with TVM, whatever its arguments
(scripts/configure_kernels.py:40-69: `topi.nn.batch_matmul`, `topi.nn.dense`, `topi.nn.conv2d` on the shapes of
:14-38).  Here an operator of a new shape is one more instantiation of a template the library already has, with
the template's default tiling:

    conv2d  [N, H, W, CO, CI, KH, KW, stride, padding]  ->  ConvF32Auto<CI, CO, H, W, KH, KW, stride, padding, N>
    bgemm   [batch, M, K, N]                            ->  GemmF32<M, N, K, BM, BN, KS, kEpiNone, 2, 1, true, batch>
    dense   [batch, in, out]                            ->  GemmF32<batch, out, in, BM, BN, KS, kEpiNone, 2, 1, true>
                                                            (weight (out, in), the reference's layout: `..._nk`)

This module writes those registrations into `<suite>/hip/operators/pairs_operators.hip` and builds them, with the
library's flags and build checks, into a kernel module of their own, `<suite>/hip/operators/libbfuse_pairs.so`
(csrc/Makefile, target `module`); `<suite>/config/modules.yaml` names it ahead of the module `build_pairs` builds
from the suite's fused kernels.  `configure --build-missing` calls it; the suite, the quick start and the
`benchmark` driver find the new operators by name once the module is loaded.

What the templates take: products of at least 16 rows and 16 columns, columns in multiples of 4 and a contracted
dimension in multiples of 16 (tiles need not divide rows or columns: the last tile overlaps its neighbour); input
channels in groups of 16 (or at most 4) and output channels in multiples of 16.  An id outside that is reported
with the reason.
"""
import os
import subprocess
from typing import Dict, List, Optional, Sequence, Tuple

import yaml

from . import configure as cfgure

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
MODULE_DIR = os.path.join("hip", "operators")
UNIT = "pairs_operators.hip"
HEADERS = ("fuse.h", "ops_conv_rect.h", "ops_gemm_f32.h")


def _tile(d: int, divisors: Sequence[int]) -> int:
    """A tile extent for a dimension of d: the first of `divisors` that divides it; where none does, or only 16
    divides a dimension above 64 (208 = 13 x 16), the largest of 64, 32, 16 that fits -- the last tile then
    overlaps its neighbour, which GemmF32 allows."""
    t = next((c for c in divisors if d % c == 0), None)
    if t is None or (t == 16 and d > 64):
        t = next(c for c in (64, 32, 16) if c <= d)
    return t


def gemm_tiling(m: int, n: int, k: int) -> Tuple[int, int, int]:
    """(BM, BN, KS) of GemmF32 for an m x n x k product: 64 rows (else 32, 16) by 64 columns (else 96, 80, 48, 32,
    16), and two or four waves over K when K is long."""
    ks = 4 if k >= 2048 and k % 64 == 0 else 2 if k >= 512 and k % 32 == 0 else 1
    return _tile(m, (64, 32, 16)), _tile(n, (64, 96, 80, 48, 32, 16)), ks


def unsupported(kernel_id: str, args) -> Optional[str]:
    """Why the library's templates cannot be instantiated for this id, or None."""
    op = cfgure.operator_of(kernel_id)
    cfgure.shapes_of(kernel_id, args)
    if op == "conv2d":
        n, h, w, co, ci, kh, kw, stride, pad = args
        if ci % 16 != 0 and ci > 4:
            return "input channels come in groups of 16, or at most 4"
        if co % 16 != 0:
            return "output channels come in multiples of 16"
        if min(n, h, w, co, ci, kh, kw) < 1 or (h - kh + 2 * pad) < 0 or (w - kw + 2 * pad) < 0:
            return "empty operand or result"
        return None
    if min(args) < 1:
        return "empty operand or result"
    m, k, n = (args[1], args[2], args[3]) if op == "bgemm" else (args[0], args[1], args[2])
    if m < 16 or n < 16:
        return "a matrix product has at least 16 rows and 16 columns (one MFMA block)"
    if n % 4 != 0:
        return "output rows are whole 16-byte chunks: columns in multiples of 4"
    if k % 16 != 0:
        return "the contracted dimension comes in multiples of 16"
    return None


def registration(kernel_id: str, args) -> Tuple[str, List[str]]:
    """(registry name, source lines) of the kernel that implements the id."""
    op = cfgure.operator_of(kernel_id)
    why = unsupported(kernel_id, args)
    if why:
        raise ValueError(f"{kernel_id} {list(args)}: {why}")
    if op == "conv2d":
        n, h, w, co, ci, kh, kw, s, p = args
        name = cfgure.candidate_names(kernel_id, args, None)[-1]
        oh, ow = (h - kh + 2 * p) // s + 1, (w - kw + 2 * p) // s + 1
        alias = f"Op_{name}"
        return name, [f"using {alias} = ConvF32Auto<{ci}, {co}, {h}, {w}, {kh}, {kw}, {s}, {p}, {n}>;",
                      f"BFUSE_KERNEL({name}, {alias}, ({{{{{n}, {ci}, {h}, {w}}}, 4}}), ({{{{{co}, {ci}, {kh}, {kw}}}, 4}}), ({{{{{n}, {co}, {oh}, {ow}}}, 4}}))"]
    if op == "bgemm":
        b, m, k, n = args
        bm, bn, ks = gemm_tiling(m, n, k)
        name = f"bgemm_f32_{b}x{m}x{k}x{n}"
        alias = f"Op_{name}"
        return name, [f"using {alias} = GemmF32<{m}, {n}, {k}, {bm}, {bn}, {ks}, kEpiNone, 2, 1, true, {b}>;",
                      f"BFUSE_KERNEL({name}, {alias}, ({{{{{b}, {m}, {k}, 1}}, 4}}), ({{{{{b}, {n}, {k}, 1}}, 4}}), ({{{{{b}, {m}, {n}, 1}}, 4}}))"]
    b, i, o = args
    bm, bn, ks = gemm_tiling(b, o, i)
    name = f"gemm_f32_{b}x{i}x{o}_nk"
    alias = f"Op_{name}"
    return name, [f"using {alias} = GemmF32<{b}, {o}, {i}, {bm}, {bn}, {ks}, kEpiNone, 2, 1, true>;",
                  f"BFUSE_KERNEL({name}, {alias}, ({{{{{b}, {i}, 1, 1}}, 4}}), ({{{{{o}, {i}, 1, 1}}, 4}}), ({{{{{b}, {o}, 1, 1}}, 4}}))"]


def source_text(ids: Dict[str, Sequence[int]]) -> str:
    """One translation unit with the kernels of `ids` ({operator id: argument list}); two ids with the same
    arguments share a kernel."""
    lines = ["// Written by bfuse_project_amd.build_operators: operators of one suite's config at the templates' default tilings."]
    lines += [f'#include "{h}"' for h in HEADERS]
    lines += ["", "using namespace bfuse;", "", "BFUSE_MODULE_PROLOGUE()", ""]
    seen = set()
    for kid, args in ids.items():
        name, reg = registration(kid, args)
        if name in seen:
            continue
        seen.add(name)
        lines.append(f"// {kid}: {list(args)}")
        lines += reg
    return "\n".join(lines) + "\n"


def name_module(suite: str, rel: str, first: bool = False) -> None:
    """Adds a module (path relative to the suite) to <suite>/config/modules.yaml, keeping what it names already."""
    os.makedirs(os.path.join(suite, "config"), exist_ok=True)
    p = os.path.join(suite, "config", "modules.yaml")
    have = []
    if os.path.exists(p):
        with open(p) as f:
            have = yaml.safe_load(f) or []
    if rel not in have:
        have = [rel] + have if first else have + [rel]
    with open(p, "w") as f:
        yaml.safe_dump(have, f)


def rebuild_and_load(suite: str, jobs: int = 8) -> Optional[str]:
    """Brings the operators' module of a suite up to date with the library's headers and loads it; None if the
    suite has none."""
    hip = os.path.join(suite, MODULE_DIR)
    if not os.path.exists(os.path.join(hip, UNIT)):
        return None
    r = subprocess.run(["make", "-C", CSRC, f"MODDIR={os.path.abspath(hip)}", f"-j{jobs}", "module"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building the operators of {suite} failed:\n{r.stdout[-3000:]}\n{r.stderr[-3000:]}")
    module = os.path.abspath(os.path.join(hip, "libbfuse_pairs.so"))
    from . import _lib
    _lib.check(_lib.lib().bfuse_load_kernels(module.encode()))
    return module


def build(suite: str, ids: Dict[str, Sequence[int]], jobs: int = 8, compile_: bool = True) -> dict:
    """Writes <suite>/hip/operators/pairs_operators.hip for `ids`, builds the operators' module and loads it into this process.
    Returns {"kernels": {id: registry name}, "file": path, "module": path or None}."""
    names = {kid: registration(kid, args)[0] for kid, args in ids.items()}     # raises for what the templates do not take
    hip = os.path.join(suite, MODULE_DIR)
    os.makedirs(hip, exist_ok=True)
    path = os.path.join(hip, UNIT)
    with open(path, "w") as f:
        f.write(source_text(ids))
    module = os.path.join(hip, "libbfuse_pairs.so")
    if not compile_:
        return {"kernels": names, "file": path, "module": None}
    r = subprocess.run(["make", "-C", CSRC, f"MODDIR={os.path.abspath(hip)}", f"-j{jobs}", "module"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building {module} failed:\n{r.stdout[-3000:]}\n{r.stderr[-3000:]}")
    name_module(suite, os.path.join(MODULE_DIR, "libbfuse_pairs.so"), first=True)
    from . import _lib
    _lib.check(_lib.lib().bfuse_load_kernels(os.path.abspath(module).encode()))
    return {"kernels": names, "file": path, "module": module}
