"""Launches registry kernels over seeded inputs a fixed number of times and prints what each takes; for use
on its own or under rocprofv3:

    python3 -m bfuse_project_amd.profile_kernels gemm_f32_512x768x768 transpose16_4096x14336 [--reps 300]
    rocprofv3 --kernel-trace --stats --output-format csv -d OUT -- python3 -m bfuse_project_amd.profile_kernels NAME ...
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d OUT -- python3 -m bfuse_project_amd.profile_kernels --copy-probe --device-fill --reps 3 --warmup 1 NAME ...

A standalone kernel runs on side 1 next to a small partner; a fused kernel runs over the two standalone
kernels it names.  Inputs: N(0, 1) data and N(0, 0.02) second operands, cast to the kernel's element type
(timing does not depend on them for fp32; a bf16 GEMM is slower on such data than on constants).
"""
import argparse

import numpy as np

import bfuse_project_amd as bf
from bfuse_project_amd.operation import fill_normal, f32_to_bf16


def _operand(seed, count, elem_bytes, std):
    if elem_bytes == 4:
        return fill_normal(seed, count, 0.0, std)
    if elem_bytes == 2:
        return f32_to_bf16(fill_normal(seed, count, 0.0, std))
    return (np.arange(count) % 251).astype(np.uint8)


def inputs_of(k, seed):
    n = [int(np.prod(s)) for s in k.shapes]
    return _operand(seed, n[0], k.elem_bytes[0], 1.0), _operand(seed + 1, n[1], k.elem_bytes[1], 0.02)


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("kernels", nargs="+")
    ap.add_argument("--reps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--device-fill", action="store_true", help="write uniform operands on the device instead of filling them on the host (operands of several GB)")
    ap.add_argument("--copy-probe", action="store_true", help="first launch a 64 MiB -> 64 MiB copy kernel: the scale of the FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.copy_probe:
        with bf.Operation("copy_f32_16777216", "bias_relu_4096") as op:
            op.upload(0, np.ones(16777216, np.float32), np.zeros(1, np.float32))
            for _ in range(5):
                op.launch("kernel1")
            op.synchronize()
    for name in args.kernels:
        k = bf.kernel_info(name)
        if k.kind == 0:
            sides, mode, fused = (name, "bias_relu_4096"), "kernel1", None
        elif k.n_sides == 2:
            sides, mode, fused = (k.sides[0], k.sides[1]), ("hfuse" if k.kind == 2 else "bfuse"), k
        else:
            raise SystemExit(f"{name}: a fusion of {k.n_sides} kernels; use profile_pair --group")
        with bf.Operation(*sides) as op:
            for side in (0, 1):
                if args.device_fill and all(e in (2, 4) for e in op.k[side].elem_bytes[:2]):
                    op.fill_uniform_device(side, 0, 0x5EED + 16 * side, -0.5, 0.5)
                    op.fill_uniform_device(side, 1, 0x5EED + 16 * side + 1, -0.5, 0.5)
                else:
                    op.upload(side, *inputs_of(op.k[side], 0x5EED + 16 * side))
            t = op.time(mode, fused, warmup=args.warmup, reps=args.reps)[0]
            q = op.time_batched(mode, fused, warmup=args.warmup, reps=args.reps)
        print(f"{name}: {float(np.mean(t)):.2f} us per launch (min {float(np.min(t)):.2f}), {q:.2f} us queued; grid {k.grid[0]} x {k.block[0]} threads", flush=True)


if __name__ == "__main__":
    main()
