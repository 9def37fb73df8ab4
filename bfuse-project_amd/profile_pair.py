"""Launches the kernels of one synthetic pair a fixed number of times, for use under rocprofv3:

    rocprofv3 --kernel-trace --stats --output-format csv -d OUT -- python3 -m bfuse_project_amd.profile_pair --pair 2
    rocprofv3 --pmc FETCH_SIZE  --output-format csv -d OUT -- python3 -m bfuse_project_amd.profile_pair --pair 2 --copy-probe
    rocprofv3 --pmc WRITE_SIZE  --output-format csv -d OUT -- python3 -m bfuse_project_amd.profile_pair --pair 2 --copy-probe

With --copy-probe a 64 MiB -> 64 MiB copy kernel is launched first (in a separate operation), so
that the same counter can be read for a kernel whose traffic is known.
Order of launches per repetition: kernel1, kernel2 (back to back on one stream), fused.
With --group NAME the kernels of a fusion of more than two (workloads.GROUPS) are launched instead:
its standalone kernels back to back, then the fused kernel.
"""
import argparse
import numpy as np

import bfuse_project_amd as bf
from bfuse_project_amd.workloads import GROUPS, HEADLINE, PAIRS


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--pair", type=int, default=2)
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--fusion", default="", help="kind[:suffix][@k1,k2]; default: the pair's headline fusion")
    ap.add_argument("--copy-probe", action="store_true")
    ap.add_argument("--group", default="", help="a fusion of more than two kernels (workloads.GROUPS) instead of a pair")
    args = ap.parse_args()
    if args.copy_probe:
        with bf.Operation("copy_f32_16777216", "bias_relu_4096") as op:
            op.upload(0, np.ones(16777216, np.float32), np.zeros(1, np.float32))
            for _ in range(args.reps):
                op.launch("kernel1")
            op.synchronize()
    if args.group:
        names, kind, suffixes, inputs = GROUPS[args.group]
        with bf.GroupOperation(names) as op:
            for i, (I, F) in enumerate(inputs()):
                op.upload(i, I, F)
            fused = op.fused(kind, suffixes[0])
            for _ in range(args.reps):
                op.launch(op.unfused())
                op.launch([(fused, tuple(range(len(names))))])
            op.synchronize()
        print(f"launched {args.reps} x [{', '.join(names)}, {fused.name}]")
        return
    pair = PAIRS[args.pair]
    k1, k2, kind, suffix = HEADLINE[args.pair]
    if args.fusion:
        spec, _, ks = args.fusion.partition("@")
        kind, _, suffix = spec.partition(":")
        if ks:
            k1, k2 = ks.split(",")
    I1, F1, I2, F2 = pair.inputs()
    with bf.Operation(k1, k2) as op:
        op.upload(0, I1, F1)
        op.upload(1, I2, F2)
        fused = op.fused(kind, suffix)
        for _ in range(args.reps):
            op.launch("serial")
            op.launch(kind, fused)
        op.synchronize()
    print(f"launched {args.reps} x [{k1}, {k2}, {fused.name}]")


if __name__ == "__main__":
    main()
