"""Launches the kernels of one synthetic pair a fixed number of times, for use under rocprofv3:

    rocprofv3 --kernel-trace --stats --output-format csv -d OUT -- python3 -m bfuse_project_amd.profile_pair --pair 2
    rocprofv3 --pmc FETCH_SIZE  --output-format csv -d OUT -- python3 -m bfuse_project_amd.profile_pair --pair 2 --copy-probe
    rocprofv3 --pmc WRITE_SIZE  --output-format csv -d OUT -- python3 -m bfuse_project_amd.profile_pair --pair 2 --copy-probe

With --copy-probe a 64 MiB -> 64 MiB copy kernel is launched first (in a separate operation), so
that the same counter can be read for a kernel whose traffic is known.
Order of launches per repetition: kernel1, kernel2 (back to back on one stream), fused.
With --clock (pair 5 only, no profiler needed) the instrumented instance of the bf16 GEMM
(`gemm_bf16_512x4096x14336_clk`: the headline kernel with clock stamps per workgroup) is run alone
and with the norm waves fused in, and the stamps are tabulated: shader clock, clocks per 64-k stage
of the K loop, and when the loops start and end on each XCD.
With --group NAME the kernels of a fusion of more than two (workloads.GROUPS) are launched instead:
its standalone kernels back to back, then the fused kernel.
"""
import argparse
import numpy as np

import bfuse_project_amd as bf
from bfuse_project_amd.workloads import GROUPS, HEADLINE, PAIRS


def clock_table(reps: int) -> str:
    """Runs the stamped GEMM (alone, then thread-fused with the norm waves) after `reps` untimed launches of the
    same kernel and tabulates the stamps of the last launch."""
    k1, k2 = "gemm_bf16_512x4096x14336_clk", "rmsnorm_rope_bf16_512x4096_w2"
    m, n, nkt, words = 512, 14336, 4096 // 64, 8
    I1, F1, I2, F2 = PAIRS[5].inputs()
    lines = []
    with bf.Operation(k1, k2) as op:
        op.upload(0, I1, F1)
        op.upload(1, I2, F2)
        for label, mode, handle in (("GEMM alone", "kernel1", None), ("GEMM + norm waves (thread-fused)", "hfuse", op.fused("hfuse"))):
            for _ in range(reps):
                op.launch(mode, handle) if handle is not None else op.launch(mode)
            op.synchronize()
            op.launch(mode, handle) if handle is not None else op.launch(mode)
            out = op.download(0)
            st = out.ravel().view(np.uint8)[m * n * 2:].view(np.uint64).reshape(-1, words).astype(np.int64)
            clk, wall, xcc = st[:, 0:3], st[:, 3:6], st[:, 6] & 15
            t0 = wall[:, 0].min()
            us = (wall - t0) / 100.0                                  # 100 MHz wall clock
            loop_us = us[:, 1] - us[:, 0]
            ghz = (clk[:, 1] - clk[:, 0]) / np.maximum(wall[:, 1] - wall[:, 0], 1) * 0.1
            per_stage = (clk[:, 1] - clk[:, 0]) / nkt
            lines.append(f"### {label}: {st.shape[0]} workgroups, {nkt} K-stages of 64, stamps of the launch after {reps} warm-up launches")
            lines.append(f"shader clock inside the K loop: median {np.median(ghz):.3f} GHz (min {ghz.min():.3f}, max {ghz.max():.3f})")
            lines.append(f"shader clocks per K-stage: median {np.median(per_stage):.0f} (min {per_stage.min():.0f}, max {per_stage.max():.0f}); "
                         f"its 896 MFMA clocks are {896 / np.median(per_stage) * 100:.0f} % of that")
            lines.append(f"K loop: median {np.median(loop_us):.2f} us (min {loop_us.min():.2f}, max {loop_us.max():.2f}); "
                         f"loop end -> last store acknowledged: median {np.median(us[:, 2] - us[:, 1]):.2f} us; "
                         f"first loop start -> last store acknowledged: {us[:, 2].max():.2f} us")
            lines.append("")
            lines.append("| XCD | workgroups | loop start, first .. last (us) | loop end, first .. last (us) | last store acknowledged (us) | clock (GHz) | clocks / stage |")
            lines.append("|---|---|---|---|---|---|---|")
            for x in sorted(set(xcc.tolist())):
                sel = xcc == x
                lines.append(f"| {x} | {int(sel.sum())} | {us[sel, 0].min():.2f} .. {us[sel, 0].max():.2f} | {us[sel, 1].min():.2f} .. {us[sel, 1].max():.2f} | "
                             f"{us[sel, 2].max():.2f} | {np.median(ghz[sel]):.3f} | {np.median(per_stage[sel]):.0f} |")
            lines.append("")
    return "\n".join(lines)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--pair", type=int, default=2)
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--fusion", default="", help="kind[:suffix][@k1,k2]; default: the pair's headline fusion")
    ap.add_argument("--copy-probe", action="store_true")
    ap.add_argument("--group", default="", help="a fusion of more than two kernels (workloads.GROUPS) instead of a pair")
    ap.add_argument("--clock", action="store_true", help="pair 5: run the clock-stamped GEMM and tabulate its stamps (use --reps 300 or more)")
    args = ap.parse_args()
    if args.clock:
        print(clock_table(args.reps))
        return
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
