"""One command from a user config to the speed-up table: the reference's scripts/quick_start.py
(`quick_start.py example -o file`, its six steps :27-160).

    python -m bfuse_project_amd.quick_start example.yaml -o OUT [--dtype f32|bf16] [--skip-missing | --build-missing] [--build-pairs] [--resident]

  reference step                                   here
  [1/6] configure test-suite (TVM kernels)         [1/3] `configure`: ids resolved against the registry (--build-missing: ids of
                                                   shapes the library lacks are instantiated from its templates and compiled)
  [2/6] generate fused kernels (hfuse, bfuse)      -- the fused kernels are in the library (OUT/config/fused.yaml lists them);
                                                   --build-pairs: `build_pairs` writes and compiles the pairs it lacks
  [3/6] generate benchmark, [4/6] make             -- the harness is the library; nothing is generated or compiled
  [5/6] profile the benchmark                      [2/3] `suite`: every pair in every mode, validated, traces under OUT/exec
                                                   (--resident: operands written and outputs compared on the device, for
                                                   operators at batch 1024 whose tensors run to GB)
  [6/6] draw profile results                       [3/3] speed-up table: OUT/summary.md, OUT/summary.json; the reference's speed-up
                                                   figure: OUT/exec_figure.png
"""
import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("example", help="example file path to generate test-suite")
    ap.add_argument("-o", dest="file", default="test-suite", help="output directory of the generated test-suite")
    ap.add_argument("--dtype", choices=("f32", "bf16"), default=None)
    ap.add_argument("--skip-missing", action="store_true", help="drop operator ids the library has no kernel for")
    ap.add_argument("--build-missing", action="store_true", help="build the operator ids the library has no kernel for from its templates (hipcc)")
    ap.add_argument("--build-pairs", action="store_true", help="build the fused kernels the library lacks for this suite's pairs (hipcc)")
    ap.add_argument("--resident", action="store_true", help="operands written and results compared on the device (operators at batch 1024)")
    args = ap.parse_args(argv)
    from . import build_pairs, configure, suite

    print("[1/3] ========================= Configure test-suite =========================", flush=True)
    if not os.path.exists(args.example):
        print(f'Given config path "{args.example}" doesn\'t exist.', file=sys.stderr)
        return 1
    try:
        r = configure.configure(args.example, args.file, args.dtype, args.skip_missing, build_missing=args.build_missing)
    except (ValueError, LookupError, FileExistsError, RuntimeError) as e:
        print(f"Error occurs while configuring '{args.file}': {e}", file=sys.stderr)
        return 1
    for kid, name in r["found"].items():
        print(f"  {kid} -> {name}")
    for kid, hint in r["missing"].items():
        print(f"  {kid}: dropped ({hint})")

    print("[2/3] ========================= Profile the benchmark =========================", flush=True)
    info = suite.load_info(os.path.join(args.file, "config", "info.yaml"))
    try:
        if args.build_pairs:
            built = build_pairs.build(args.file)
            print(f"  built {len(built['kernels'])} fused kernels", flush=True)
        build_pairs.load_suite_modules(args.file)
        rows = suite.run_suite(info, args.file, validate=True, resident=args.resident)
    except Exception as e:   # a failed validation or a device error ends the run, as the reference's check=True does
        print(f"Error occurs while profiling the benchmark: {e}", file=sys.stderr)
        return 1

    print("[3/3] ========================= Results =========================", flush=True)
    with open(os.path.join(args.file, "summary.json"), "w") as f:
        json.dump(rows, f, indent=1)
    md = suite.to_markdown(rows)
    with open(os.path.join(args.file, "summary.md"), "w") as f:
        f.write(md)
    print(md)
    try:      # the reference's [6/6]: its speed-up figure (profile/exec_figure.png)
        print(suite.draw_speedup_figure(rows, os.path.join(args.file, "exec_figure.png")))
    except ImportError:
        pass
    return 0


if __name__ == "__main__":
    sys.exit(main())
