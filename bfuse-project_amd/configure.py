"""Suite configuration from the reference's user config: the host-side half of
scripts/configure_kernels.py (:150-166 get_fusion_info, :229-320 get_test_suite).

The reference reads `FusionSet` (two `Set` lists of operator ids) and `KernelInfo` (id -> argument
list; the id's prefix names the operator: `dense` = (batch, in, out), `conv2d` = (N, H, W, CO, CI, KH,
KW, stride, padding), `bgemm` = (batch, M, K, N); :14-38), generates one kernel per id with TVM and
writes `<out>/cuda/kernels.cu` and `<out>/config/{kernels,fusions,info}.yaml`.  Here kernels are not
generated: every id is resolved against the library's registry of hand-written gfx950 kernels, whose
shapes are compile-time, and the same three config files are written for what resolved:

    python -m bfuse_project_amd.configure example.yaml -o OUT [--dtype f32|bf16] [--skip-missing | --build-missing]

Arithmetic and weight layout are part of what an id resolves to, and are written down per id: by default
every id resolves to an fp32 kernel, the reference's arithmetic; `--dtype bf16` takes the bf16 kernel where
the library holds one and says which ids stayed fp32.  The reference's `dense` weight is (out, in)
(:21-26).  The bf16 GEMMs take it like that; the fp32 GEMMs take [in, out], so a weight in the reference's
layout goes through the library's `transpose32_<out>x<in>` kernel once when it is loaded -- `info.yaml`
names that kernel, and resolution fails if a kernel's registered shapes are not the reference's shapes up
to that one stated transposition.

  OUT/config/kernels.yaml   id -> {KernelName (registry name), HasBarriers, GridDim, BlockDim, Reg, ExecTime}
                            in the fuser's schema (horizontal-fuser/include/fuse/Utils.h:70-112); launch shape and
                            barrier flag are the kernel's own, Reg is the reference's don't-care 32 unless a
                            device is present
  OUT/config/fusions.yaml   every (set 0, set 1) pair as {File, Kernels}; File names the library
  OUT/config/info.yaml      the suite description for `python -m bfuse_project_amd.suite`: the two sets
                            with registry names, the user's KernelInfo block kept beside them, and `Resolved`:
                            id -> {kernel, dtype, weight_layout, weight_transpose}
  OUT/config/fused.yaml     for every pair, the fused kernels the library holds for it

An id no registry kernel matches is reported with the lines that would instantiate it; the run then
fails (exit status 1) unless --skip-missing drops such ids from the sets, or --build-missing writes those
instantiations (the templates' default tilings) into OUT/hip/operators/, compiles them into a kernel module of
the suite and resolves the ids against it (build_operators: the counterpart of the reference generating a
kernel for whatever arguments an id has).
"""
import argparse
import os
import sys
from typing import Dict, List, Optional, Tuple

import yaml

OPERATORS = ("bgemm", "conv2d", "dense")     # configure_kernels.py:176-187


def operator_of(kernel_id: str) -> str:
    for op in OPERATORS:
        if kernel_id.startswith(op):
            return op
    raise ValueError(f"{kernel_id}: function and schedule with given kernel's name do not exist "
                     f"(ids start with one of {', '.join(OPERATORS)})")


def shapes_of(kernel_id: str, args) -> Tuple[tuple, tuple, tuple]:
    """(data, weight, output) shapes as the reference computes them (configure_kernels.py:14-38)."""
    op = operator_of(kernel_id)
    want = {"dense": 3, "bgemm": 4, "conv2d": 9}[op]
    if not isinstance(args, (list, tuple)) or len(args) != want or not all(isinstance(a, int) and a >= 0 for a in args):
        raise ValueError(f"{kernel_id}: {op} takes {want} non-negative integers, got {args!r}")
    if op == "dense":
        b, i, o = args
        return (b, i), (o, i), (b, o)
    if op == "bgemm":
        b, m, k, n = args
        return (b, m, k), (b, n, k), (b, m, n)
    n, h, w, co, ci, kh, kw, stride, pad = args
    if stride < 1:
        raise ValueError(f"{kernel_id}: stride must be at least 1")
    return (n, ci, h, w), (co, ci, kh, kw), (n, co, (h - kh + 2 * pad) // stride + 1, (w - kw + 2 * pad) // stride + 1)


def candidate_names(kernel_id: str, args, dtype: Optional[str]) -> List[str]:
    """Registry names that implement the operator at exactly these arguments, in order of preference:
    fp32 (the reference's arithmetic) unless bf16 is asked for, then bf16 first and fp32 behind it."""
    op = operator_of(kernel_id)
    shapes_of(kernel_id, args)   # validates
    types = ["bf16", "f32"] if dtype == "bf16" else ["f32"]
    if op == "dense":
        b, i, o = args
        # (`..._nk`: an fp32 kernel that takes the weight as the reference stores it, (out, in): build_operators)
        return [n for t in types for n in ([f"gemm_{t}_{b}x{i}x{o}"] + ([f"gemm_f32_{b}x{i}x{o}_nk"] if t == "f32" else []))]
    if op == "conv2d":
        n, h, w, co, ci, kh, kw, stride, pad = args
        names = []
        for t in types:
            if n != 1:                                               # a batch is part of the name
                names.append(f"conv{kh}x{kw}s{stride}p{pad}_{t}_{n}x{ci}x{h}x{w}_{co}")
                continue
            if (kh, kw, stride, pad) == (3, 3, 1, 1):
                names.append(f"conv3x3_{t}_{ci}x{h}x{w}_{co}")       # the kernel tuned for this case, where instantiated
            names.append(f"conv{kh}x{kw}s{stride}p{pad}_{t}_{ci}x{h}x{w}_{co}")
        return names
    b, m, k, n = args
    return [f"bgemm_{t}_{b}x{m}x{k}x{n}" for t in types]


# kernel families whose dense weight is stored [in, out] (= [K, N]) instead of the reference's (out, in): the
# fp32 GEMM sides (csrc/ops_gemm_f32*.h); the bf16 GEMM takes (out, in) as it is
WEIGHT_IS_IN_OUT = {"gemm_f32": True, "gemm_bf16": False}


def _dims(shape) -> tuple:
    """A shape without its padding of trailing ones."""
    d = [int(x) for x in shape]
    while len(d) > 1 and d[-1] == 1:
        d.pop()
    return tuple(d)


def describe(kernel_id: str, args, kernel, registry) -> dict:
    """What the id resolved to: kernel, arithmetic, weight layout.  The kernel's registered shapes must be the
    reference's (shapes_of), except that a dense weight may be registered transposed -- [in, out] instead of
    (out, in) -- when the library also holds the kernel that transposes it; anything else is an error."""
    data, weight, out = shapes_of(kernel_id, args)
    have = [_dims(sh) for sh in kernel.shapes]
    want = [_dims(data), _dims(weight), _dims(out)]
    dtype = {4: "f32", 2: "bf16"}.get(kernel.elem_bytes[0], f"{kernel.elem_bytes[0]} bytes")
    if have[0] != want[0] or have[2] != want[2]:
        raise ValueError(f"{kernel_id}: {kernel.name} is registered for data {have[0]} -> {have[2]}, the id asks for {want[0]} -> {want[2]}")
    info = {"kernel": kernel.name, "dtype": dtype, "weight_layout": "reference", "weight_transpose": None}
    if operator_of(kernel_id) == "dense" and not kernel.name.endswith("_nk") and WEIGHT_IS_IN_OUT.get(kernel.name.split("_")[0] + "_" + dtype, False):
        # the kernel family takes [in, out]; a square weight has the same shape either way, so the family decides
        if have[1] != want[1][::-1]:
            raise ValueError(f"{kernel_id}: {kernel.name} takes a weight of shape {have[1]}, [in, out] of the id's is {want[1][::-1]}")
        tname = f"transpose32_{want[1][0]}x{want[1][1]}"
        if tname not in registry:
            raise ValueError(f"{kernel_id}: {kernel.name} takes its weight as [in, out] {have[1]} (the reference's is (out, in)) and the library has no {tname}")
        info.update(weight_layout="[in, out]: the reference's (out, in) weight transposed once on load", weight_transpose=tname)
        return info
    if have[1] != want[1]:
        raise ValueError(f"{kernel_id}: {kernel.name} takes a weight of shape {have[1]}, the id's is {want[1]}")
    return info


def instantiation_hint(kernel_id: str, args) -> str:
    op = operator_of(kernel_id)
    if op == "dense":
        b, i, o = args
        return (f"using Dense = GemmF32Dma<{b}, {o}, {i}, BM, BN, 4>;  BFUSE_KERNEL(gemm_f32_{b}x{i}x{o}, Dense, "
                f"({{{{{b}, {i}, 1, 1}}, 4}}), ({{{{{i}, {o}, 1, 1}}, 4}}), ({{{{{b}, {o}, 1, 1}}, 4}}))  in csrc/kernels_*.hip")
    if op == "conv2d":
        n, h, w, co, ci, kh, kw, stride, pad = args
        if ci % 16 != 0 and ci > 4:
            return "the library's convolutions take input channels in groups of 16, or at most 4 (csrc/ops_conv_general.h, ops_conv_rect.h)"
        batch = f"{n}x" if n != 1 else ""
        return (f"using Conv = ConvF32Auto<{ci}, {co}, {h}, {w}, {kh}, {kw}, {stride}, {pad}, {n}>;  "
                f"BFUSE_KERNEL(conv{kh}x{kw}s{stride}p{pad}_f32_{batch}{ci}x{h}x{w}_{co}, Conv, ...)  in csrc/kernels_*.hip")
    b, m, k, n = args
    return (f"using Bgemm = GemmF32<{m}, {n}, {k}, BM, BN, KS, kEpiNone, 2, 1, true, {b}>;  BFUSE_KERNEL(bgemm_f32_{b}x{m}x{k}x{n}, Bgemm, "
            f"({{{{{b}, {m}, {k}, 1}}, 4}}), ({{{{{b}, {n}, {k}, 1}}, 4}}), ({{{{{b}, {m}, {n}, 1}}, 4}}))  in csrc/kernels_*.hip")


def load_user_config(path: str) -> dict:
    with open(path) as f:
        doc = yaml.safe_load(f)
    if not isinstance(doc, dict) or "FusionSet" not in doc or "KernelInfo" not in doc:
        raise ValueError("the config needs a FusionSet and a KernelInfo block")
    sets = doc["FusionSet"]
    if not isinstance(sets, list) or len(sets) != 2:
        raise ValueError("Number of fusion sets are only 2.")            # configure_kernels.py:155-157
    for s in sets:
        if not isinstance(s, dict) or not isinstance(s.get("Set"), list):
            raise ValueError("every FusionSet entry needs a 'Set' list")
        s["Set"] = [k for k in s["Set"] if k is not None]               # the examples ship with one empty item
        for k in s["Set"]:
            if k not in doc["KernelInfo"]:
                raise ValueError(f"{k} is in a fusion set but has no KernelInfo entry")
    if not isinstance(doc["KernelInfo"], dict):
        raise ValueError("KernelInfo must map ids to argument lists")
    return doc


def resolve(doc: dict, registry: Dict[str, object], dtype: Optional[str] = None):
    """({id: registry kernel}, {id: hint}) for every id the two sets name.  A kernel whose registered shapes are
    not the id's (up to the stated weight transposition of fp32 dense kernels) raises ValueError."""
    found, missing = {}, {}
    for s in doc["FusionSet"]:
        for kid in s["Set"]:
            if kid in found or kid in missing:
                continue
            args = doc["KernelInfo"][kid]
            hit = next((registry[n] for n in candidate_names(kid, args, dtype) if n in registry), None)
            if hit is not None:
                describe(kid, args, hit, registry)      # shapes checked here, before anything is written
                found[kid] = hit
            else:
                missing[kid] = instantiation_hint(kid, args)
    return found, missing


def configure(path: str, out: str, dtype: Optional[str] = None, skip_missing: bool = False, registry=None,
              build_missing: bool = False) -> dict:
    """Writes OUT/config/*.yaml and returns {"found", "missing", "pairs", "fused"}.  `build_missing`: the ids no
    kernel implements are instantiated from the library's templates, built into OUT/hip/operators/ and loaded."""
    from . import config as cfg
    own_registry = registry is None
    if own_registry:
        from .operation import list_kernels
        registry = {k.name: k for k in list_kernels()}
    doc = load_user_config(path)
    if os.path.exists(out):
        raise FileExistsError(f'"{out}" already exists.')                # configure_kernels.py:239-241
    found, missing = resolve(doc, registry, dtype)
    built = {}
    if missing and build_missing:
        if not own_registry:
            raise ValueError("build_missing works on the library's own registry")
        from . import build_operators
        try:
            built = build_operators.build(out, {kid: doc["KernelInfo"][kid] for kid in missing})["kernels"]
        except Exception:
            import shutil
            shutil.rmtree(out, ignore_errors=True)       # nothing half-configured is left behind
            raise
        registry = {k.name: k for k in list_kernels()}
        found, missing = resolve(doc, registry, dtype)
    if missing and not skip_missing:
        lines = [f"  {kid} {doc['KernelInfo'][kid]}: {hint}" for kid, hint in missing.items()]
        raise LookupError("no kernel of the library implements:\n" + "\n".join(lines))
    sets = [[k for k in s["Set"] if k in found] for s in doc["FusionSet"]]
    if not sets[0] or not sets[1]:
        raise LookupError("a fusion set is empty" + (" after dropping the ids the library has no kernel for" if missing else ""))
    config_dir = os.path.join(out, "config")
    os.makedirs(config_dir, exist_ok=True)

    infos = {}
    for kid, k in found.items():
        infos[kid] = cfg.KernelInfo(k.name, bool(k.has_barriers), tuple(k.grid), tuple(k.block), k.regs if k.regs > 0 else 32)
    cfg.dump_kernels_yaml(infos, os.path.join(config_dir, "kernels.yaml"))

    pairs = [(a, b) for a in sets[0] for b in sets[1]]                    # configure_kernels.py:159-163
    with open(os.path.join(config_dir, "fusions.yaml"), "w") as f:
        yaml.safe_dump([{"File": "libbfuse_rt.so", "Kernels": [a, b]} for a, b in pairs], f, sort_keys=False)

    fused = {}
    for a, b in pairs:
        ka, kb = found[a].name, found[b].name
        fused[f"{a} + {b}"] = sorted(k.name for k in registry.values() if k.kind in (1, 2, 3) and tuple(k.sides[:2]) == (ka, kb) and k.n_sides == 2)
    with open(os.path.join(config_dir, "fused.yaml"), "w") as f:
        yaml.safe_dump(fused, f, sort_keys=False)

    resolved = {kid: describe(kid, doc["KernelInfo"][kid], found[kid], registry) for kid in found}
    info = {"FusionSet": [{"Set": [found[k].name for k in s]} for s in sets],
            "KernelInfo": {kid: list(doc["KernelInfo"][kid]) for kid in found},
            "Resolved": resolved}
    with open(os.path.join(config_dir, "info.yaml"), "w") as f:
        yaml.safe_dump(info, f, sort_keys=False)
    return {"found": {k: v.name for k, v in found.items()}, "missing": missing, "pairs": pairs, "fused": fused, "resolved": resolved,
            "built": built}


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("config", help="config file path for generate test suite")
    ap.add_argument("-o", dest="file", default="test-suite", help="output directory of the generated suite configuration")
    ap.add_argument("--dtype", choices=("f32", "bf16"), default=None,
                    help="arithmetic type to resolve to: f32 (default, the reference's) or bf16 where the library holds a bf16 kernel (the others stay f32 and are listed)")
    ap.add_argument("--skip-missing", action="store_true", help="drop ids the library has no kernel for instead of failing")
    ap.add_argument("--build-missing", action="store_true", help="instantiate the ids the library has no kernel for from its templates and compile them into a module of the suite (hipcc)")
    args = ap.parse_args(argv)
    if not os.path.exists(args.config):
        print(f'Given config path "{args.config}" doesn\'t exist.', file=sys.stderr)
        return 1
    try:
        r = configure(args.config, args.file, args.dtype, args.skip_missing, build_missing=args.build_missing)
    except (ValueError, LookupError, FileExistsError, RuntimeError) as e:
        print(f"configure: {e}", file=sys.stderr)
        return 1
    for kid, d in r["resolved"].items():
        layout = f", weight {d['weight_layout']} ({d['weight_transpose']})" if d["weight_transpose"] else ""
        print(f"{kid} -> {d['kernel']}  [{d['dtype']}{layout}]")
    if args.dtype == "bf16":
        kept = [kid for kid, d in r["resolved"].items() if d["dtype"] != "bf16"]
        if kept:
            print(f"no bf16 kernel, resolved to f32: {', '.join(kept)}", file=sys.stderr)
    for kid, hint in r["missing"].items():
        print(f"{kid}: dropped, no kernel ({hint})", file=sys.stderr)
    for kid, name in r["built"].items():
        print(f"{kid}: built {name}")
    print(f"{len(r['pairs'])} pairs, {sum(1 for v in r['fused'].values() if v)} with a fused kernel; wrote {os.path.join(args.file, 'config')}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
