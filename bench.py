#!/usr/bin/env python3
"""Headline benchmark: the five fused pairs on one MI355X, each against the same two kernels
launched back to back.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--pair N] [--fusion SPEC] [--no-cpu] [--no-power-check]

A step is one launch of a fused kernel over device-resident synthetic inputs.  By default all
five pairs are measured in one run (the reference profiles its whole pair matrix,
scripts/profile_test_suite.py:13-47,130-139); the top-level figures of the JSON line are pair 5
(Llama-3-8B shapes: bf16 GEMM [512x4096].[14336x4096]^T fused with RMSNorm+RoPE), the largest
configuration, and `pairs` holds the same figures for every pair.  Where a configuration names a
fused form that is not the fastest on this chip (pair 3: 1:1 zig-zag; pair 5: block fusion), that
kernel is timed too and reported beside the measured one.  `--pair N` measures one pair only
and puts it at the top level.

`--fusion` selects the fused variant: empty = the pair's headline kernel; `auto` = the tuner's choice
(static footprint rule, then timed candidate plans on the pair's run-time-plan kernel, then the
compile-time kernel with that dispatch); `kind[:suffix][@k1,k2]` pins one (with --pair).

Prints ONE JSON line and exits non-zero if any fused output differs from the unfused kernels.
Per pair:
  fused_us          the fused kernel's GPU-side duration in microseconds: mean over the K timed
                    launches of a SECOND pass (after the baselines have run), from the start/end
                    timestamps of each dispatch on the launch stream; the first pass is beside it
  back_to_back_us   first start -> second end of the two unfused kernels on one stream
  serial_sum_us     sum of the two unfused kernel durations (the reference's "serial",
                    scripts/analyze_test_suite.py:425-428)
  batched_*_us      wall-clock microseconds per launch with K launches queued back to back
                    (includes dispatch gaps, lets consecutive launches overlap their ramp-up);
                    fused_over_back_to_back is the ratio of these queued figures
  best_unfused      the fastest standalone kernels the library holds for the two operators (every
                    registered tiling / schedule of each is timed queued), those two queued back to back,
                    and the fused kernel's queued time over that: the baseline a user would really run
  roofline          algorithmic flops (or bytes) of the pair / fused duration vs the MI355X peak;
                    `traffic` is HBM bytes per launch from the rocprofv3 --pmc summary named in
                    `traffic_source` (not measured by this run); `same_kernel_constant_operands` (pairs with a
                    matrix-core bound): the same fused kernel timed over all-ones contraction inputs -- same
                    instructions and traffic, no operand bits toggling -- i.e. what the code sustains when the
                    chip's power management is not holding the clock down for the data
Top level only:
  groups            fusions of more than two kernels (one: the fp32 QKV GEMM, LayerNorm and causal softmax
                    as one block-fused kernel) against their standalone kernels queued back to back
  cpu_baseline      the OpenMP CPU reference (oracle/) timed on this host's cores
  measured_ceilings what this chip sustains in this run, beside the published peaks `roofline.peak` divides by:
                    the library's 64 MiB -> 64 MiB copy kernel (GB/s; also `hbm_copy_GBps`) and its MFMA-only
                    kernels, bf16 and fp32, with operands that toggle bits and no memory traffic (TFLOP/s);
                    each pair's `roofline.measured_peak` / `frac_of_measured_peak` use the one of its bound
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402


# launches per unfused baseline and per queued figure when --steps is smaller (see measure())
BASELINE_MIN_REPS = 500
# queued (wall-clock) runs per figure of the fused / back-to-back ratio; the median is reported
QUEUED_ROUNDS = 5


def cpu_baseline(pair_number, I1, F1, I2, F2, passes=5):
    """Times the CPU oracle (the checker, not the product) on this host: best of `passes`."""
    from oracle import oracle as orf
    from tests import oracle_cases

    def best(f):
        b = None
        for _ in range(passes):
            t0 = time.perf_counter()
            f()
            dt = time.perf_counter() - t0
            b = dt if b is None else min(b, dt)
        return b

    if pair_number == 5:
        # The bf16 GEMM is 60 GFLOP in double on the CPU: ~1.5 s on a GPU box's host cores, minutes on a
        # small host.  A 1/64 strided sample of its outputs (64 rows x 1792 columns over the full K) is
        # timed first; if that projects to a few seconds the whole GEMM is timed, otherwise the sample is
        # scaled.  The RMSNorm+RoPE side is timed in full either way.
        from bfuse_project_amd.workloads import unpack_norm_rope_operand
        A, Wt = I1.reshape(512, 4096), F1.reshape(14336, 4096)
        As, Ws = np.ascontiguousarray(A[3::8]), np.ascontiguousarray(Wt[5::8])
        w, cosv, sinv = unpack_norm_rope_operand(F2, 512, 4096, 128)
        t_s = best(lambda: orf.gemm_bf16(As, Ws, b_is_nk=True))
        t_n = best(lambda: orf.rmsnorm_rope_bf16(I2.reshape(512, 4096), w, cosv, sinv, heads=32, eps=1e-5))
        if t_s * 64 <= 5.0:
            t_g = best(lambda: orf.gemm_bf16(A, Wt, b_is_nk=True))
            total = t_g + t_n
            sample = (f"the whole pair: GEMM 512x4096x14336 in full ({t_g * 1e3:.0f} ms; its 1/64 output sample alone {t_s * 1e3:.1f} ms), "
                      f"RMSNorm+RoPE in full ({t_n * 1e3:.2f} ms); OpenMP, double accumulation, best of {passes}")
        else:
            total = t_s * 64 + t_n
            sample = (f"GEMM timed on a 1/64 strided sample of the outputs (64x1792 over K=4096, {t_s * 1e3:.1f} ms) and "
                      f"scaled x64; RMSNorm+RoPE in full ({t_n * 1e3:.2f} ms); best of {passes}")
    else:
        total = best(lambda: oracle_cases.expected(pair_number, I1, F1, I2, F2))
        sample = f"best of {passes} full passes of pair {pair_number} (both operators, OpenMP, double accumulation)"
    return {"value": round(total * 1e6, 1), "unit": "us", "cores": orf.num_threads(), "kind": "port", "sample": sample}


def hbm_copy_rate(reps=50):
    """GB/s of the library's 64 MiB -> 64 MiB copy kernel (the PMC calibration kernel), from its
    dispatch timestamps: a measured ceiling for streaming kernels on this box."""
    import bfuse_project_amd as bf
    with bf.Operation("copy_f32_16777216", "bias_relu_4096") as op:
        op.upload(0, np.ones(16777216, np.float32), np.zeros(1, np.float32))
        t = op.time("kernel1", warmup=5, reps=reps)[0]
    return 2 * 16777216 * 4 / float(np.mean(t)) * 1e-3


# the library's MFMA-only kernels (csrc/ops_ceiling.h): name and flops per launch, by arithmetic type
MFMA_STREAMS = {"bf16": ("mfma_stream_bf16_2000", 256 * 8 * 14 * 2000 * 16384.0),
                "f32": ("mfma_stream_f32_1000", 256 * 8 * 14 * 1000 * 2048.0)}


def mfma_stream_rate(dtype, reps=100):
    """TFLOP/s of a dense stream of independent MFMAs of this type with operands that toggle bits and no
    memory traffic (two waves per SIMD on every CU): what the matrix cores sustain at the clock the chip
    grants them in this run -- a measured ceiling beside the published peak."""
    import bfuse_project_amd as bf
    name, flops = MFMA_STREAMS[dtype]
    with bf.Operation(name, "bias_relu_4096") as op:
        op.upload(0, np.zeros(1, np.float32), np.zeros(1, np.float32))
        # 100 launches of 0.4-0.6 ms: long enough for the power management to settle (the first few
        # milliseconds of a burst run faster than what the chip then sustains)
        t = op.time("kernel1", warmup=20, reps=reps)[0]
    return flops / float(np.mean(t[reps // 2:])) * 1e-6


def measured_ceilings():
    return {"hbm_copy_GBps": round(hbm_copy_rate(), 1),
            "mfma_bf16_TFLOPs": round(mfma_stream_rate("bf16"), 1),
            "mfma_f32_TFLOPs": round(mfma_stream_rate("f32"), 1)}


def pick_fusion(number, spec):
    """(k1, k2, kind, suffix, note) for a pair under --fusion `spec`."""
    import bfuse_project_amd as bf
    from bfuse_project_amd import tuner
    from bfuse_project_amd.workloads import HEADLINE, PAIRS, RT_SIDES, CONFIG_KINDS
    k1, k2, kind, suffix = HEADLINE[number]
    if not spec:
        return k1, k2, kind, suffix, {"mode": "headline"}
    if spec != "auto":
        s, _, ks = spec.partition("@")
        kind, _, suffix = s.partition(":")
        if ks:
            k1, k2 = ks.split(",")
        return k1, k2, kind, suffix, {"mode": "pinned"}
    # auto: the footprint rule picks the kind; for block fusion the candidate plans are timed on the
    # pair's run-time-plan kernel and the winner is looked up among the compile-time kernels
    pair = PAIRS[number]
    I1, F1, I2, F2 = pair.inputs()
    a, b = bf.kernel_info(k1), bf.kernel_info(k2)
    with bf.Operation(*RT_SIDES[number]) as op:
        choice = tuner.static_plan(bf.kernel_info(k1), bf.kernel_info(k2), kinds=CONFIG_KINDS[number])
        note = {"mode": "auto", "static": {k: v for k, v in choice.items() if k != "static"}, "footprint": choice["static"]}
        if choice["kind"] == "bfuse":
            op.upload(0, I1, F1)
            op.upload(1, I2, F2)
            rows = [r for r in tuner.autotune(op, warmup=20, reps=100) if not r["persistent"]]
            best = rows[0]
            note["timed"] = [{"label": r["label"], "us": round(r["us_mean"], 2)} for r in rows[:4]]
            choice = {"kind": "bfuse", "pattern": best["pattern"], "p0": best["p0"], "p1": best["p1"]}
    h = tuner.find_variant(a, b, choice)
    if h is None:   # the winner has no compile-time instantiation: keep the footprint rule's kernel
        h = tuner.find_variant(a, b, tuner.static_plan(a, b, kinds=CONFIG_KINDS[number]))
        note["fallback"] = "timed winner is not instantiated at compile time"
    if h is None:
        return k1, k2, kind, suffix, {**note, "fallback": "no built kernel realises the choice; headline kept"}
    hk = "hfuse" if h.kind == 2 else "bfuse"
    sfx = h.name.split("_fused_" + hk, 1)[1]
    note["is_headline"] = (hk, sfx) == (kind, suffix)
    return k1, k2, hk, sfx, note


def best_unfused(k1, k2, inputs, R, BW, b_ser, b_k1, b_k2):
    """Queued time of the fastest standalone kernels for the two operators of a pair.  Every registered
    alternative of each side is timed queued on its own; if the fastest ones are not (k1, k2), that pair is
    then timed queued back to back (median of three runs).  b_ser / b_k1 / b_k2: the figures already
    measured for (k1, k2)."""
    import bfuse_project_amd as bf
    from bfuse_project_amd.workloads import BASELINE_NOTES, standalone_alternatives
    I1, F1, I2, F2 = inputs
    alone = [{k1: b_k1}, {k2: b_k2}]
    for side, (mine, partner) in enumerate(((k1, k2), (k2, k1))):
        for alt in standalone_alternatives(mine):
            if alt == mine:
                continue
            pair = (alt, partner) if side == 0 else (partner, alt)
            with bf.Operation(*pair) as op:
                op.upload(0, I1, F1)
                op.upload(1, I2, F2)
                alone[side][alt] = op.time_batched("kernel1" if side == 0 else "kernel2", warmup=BW, reps=R)
    pick = [min(d, key=d.get) for d in alone]
    out = {"kernel1": pick[0], "kernel2": pick[1],
           "alone_us": [{k: round(v, 3) for k, v in d.items()} for d in alone],
           "is_the_fused_kernels_own_pair": (pick[0], pick[1]) == (k1, k2)}
    if (pick[0], pick[1]) == (k1, k2):
        out["batched_back_to_back_us"] = round(b_ser, 3)
    else:
        with bf.Operation(pick[0], pick[1]) as op:
            op.upload(0, I1, F1)
            op.upload(1, I2, F2)
            q = [op.time_batched("serial", warmup=BW, reps=R) for _ in range(3)]
        out["batched_back_to_back_us"] = round(float(np.median(q)), 3)
    notes = [f"{k}: {BASELINE_NOTES[k]}" for k in pick if k in BASELINE_NOTES]
    if notes:
        out["notes"] = notes
    return out


def measure(number, K, W, spec, ceilings, power_check=True):
    import bfuse_project_amd as bf
    from bfuse_project_amd import tuner
    from bfuse_project_amd.workloads import PAIRS, measured_traffic, TRAFFIC_SOURCE, CONFIG_KINDS, BESIDE, FLOORS

    pair = PAIRS[number]
    k1, k2, kind, suffix, note = pick_fusion(number, spec)
    inputs = pair.inputs()
    I1, F1, I2, F2 = inputs
    with bf.Operation(k1, k2) as op:
        dev = bf.operation.device_name()
        op.upload(0, I1, F1)
        op.upload(1, I2, F2)
        fused = op.fused(kind, suffix)
        # what the footprint rule alone selects, and whether the measured kernel is that choice
        st = tuner.static_plan(op.k[0], op.k[1], kinds=CONFIG_KINDS[number])
        sv = tuner.find_variant(op.k[0], op.k[1], st)
        chooser = {"kind": st["kind"], "pattern": st["pattern"], "p0": st["p0"],
                   "wg_per_cu": list(st["static"]["wg_per_cu"]), "kernel": sv.name if sv else None,
                   "is_measured_kernel": bool(sv and sv.name == fused.name)}

        # correctness inside the bench: fused output must equal the unfused kernels bit for bit
        op.zero_outputs()
        op.launch("serial")
        U1, U2 = op.download(0), op.download(1)
        op.zero_outputs()
        op.launch(kind, fused)
        Q1, Q2 = op.download(0), op.download(1)
        bit_exact = bool(np.array_equal(U1.view(np.uint8), Q1.view(np.uint8)) and
                         np.array_equal(U2.view(np.uint8), Q2.view(np.uint8)))

        # GPU-side durations (dispatch timestamps).  The fused kernel: W warm-up + exactly K timed
        # launches per pass.  The unfused baselines are figures of their own and take R = max(K, 500)
        # launches, so that a short run (K = 20 is one millisecond of work) still compares against
        # baselines with usable statistics -- and the reported fused pass, which follows them, finds the
        # chip at the clock a busy GPU runs at instead of the one it idles at.
        R = max(K, BASELINE_MIN_REPS)
        t_f1 = op.time(kind, fused, warmup=W, reps=K)[0]
        t_par = op.time("parallel", warmup=W, reps=R)[0]     # meets the host after every repetition: run first
        t_ser, t_a, t_b = op.time("serial", warmup=W, reps=R)
        t_f = op.time(kind, fused, warmup=W, reps=K)[0]     # the reported pass: after the baselines
        fused_us = float(t_f.mean())

        # the timed region of the contract: W untimed, then exactly K steps between two syncs
        for _ in range(W):
            op.launch(kind, fused)
        op.synchronize()
        t0 = time.perf_counter()
        for _ in range(K):
            op.launch(kind, fused)
        op.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / K

        # queued figures: fused and unfused alike, R untimed launches of the same thing and then R timed
        # ones (a ratio of two like runs; whichever came first would otherwise meet the colder chip)
        # Each figure is the median of QUEUED_ROUNDS such runs, fused and unfused taking turns: a single
        # wall-clock run of R launches moves by 2 % with whatever else the host and the chip do, and pair 2's
        # ratio sits 1.5 % under the 0.9 it is compared with.
        BW = max(W, R)
        q_f, q_ser = [], []
        for _ in range(QUEUED_ROUNDS):
            q_f.append(op.time_batched(kind, fused, warmup=BW, reps=R))
            q_ser.append(op.time_batched("serial", warmup=BW, reps=R))
        b_f, b_ser = float(np.median(q_f)), float(np.median(q_ser))
        b_k1 = op.time_batched("kernel1", warmup=BW, reps=R)
        b_k2 = op.time_batched("kernel2", warmup=BW, reps=R)
        # The same three things replayed from a HIP graph (20 repetitions captured as one graph: the two kernels
        # as dependent nodes / as independent nodes between a fork and a join / the fused kernel): what is left of
        # each figure when the host's launch path is out of it.  The unfused pair as a graph is the strongest
        # unfused baseline a caller has.
        GC, GR = 20, max(3, R // 20)
        try:
            for mode, f in ((kind, fused), ("serial", None), ("parallel", None)):
                op.time_graph(mode, f, chain=GC, reps=1)
            graph = {"chain": GC,
                     "fused_us": round(float(np.median([op.time_graph(kind, fused, chain=GC, reps=GR) for _ in range(3)])), 3),
                     "back_to_back_us": round(float(np.median([op.time_graph("serial", chain=GC, reps=GR) for _ in range(3)])), 3),
                     "two_branches_us": round(float(np.median([op.time_graph("parallel", chain=GC, reps=GR) for _ in range(3)])), 3)}
            graph["fused_over_back_to_back"] = round(graph["fused_us"] / graph["back_to_back_us"], 4)
            graph["fused_over_best_unfused_graph"] = round(graph["fused_us"] / min(graph["back_to_back_us"], graph["two_branches_us"]), 4)
        except bf._lib.BfuseError as e:      # refused under rocprofv3 (its tracing does not survive graph launches)
            graph = {"skipped": str(e)}

        # The same fused kernel over constant operands (every element of the contraction's two inputs = 1):
        # the same instructions and the same memory traffic, but no bits toggle in the matrix cores'
        # operands, so the power management grants a higher clock.  What this reads is what the kernel's
        # code sustains; the distance to `fused_us` is what the data costs in power on this chip.
        const = None
        if pair.bound == "mfma" and power_check:
            side = 0 if k1.startswith(("gemm", "conv")) else 1
            ones = [np.full(x.shape, 0x3f80, np.uint16) if x.dtype == np.uint16 else np.ones(x.shape, np.float32)
                    for x in (inputs[2 * side], inputs[2 * side + 1])]
            op.upload(side, *ones)
            t_c = op.time(kind, fused, warmup=BW, reps=R)[0]
            const = {"fused_us": round(float(t_c.mean()), 3), "contraction_side": side + 1,
                     "achieved": round(pair.flops / float(t_c.mean()) * 1e-6, 2),
                     "frac": round(pair.flops / float(t_c.mean()) * 1e-6 / pair.peak, 4)}
            op.upload(side, inputs[2 * side], inputs[2 * side + 1])

    # The honest baseline: for each side, the fastest standalone kernel the library holds for that operator
    # at that shape (another tiling or schedule of it), found by timing them queued, and then those two
    # queued back to back.  The headline sides are the kernels the fusion was built from, which is not
    # always the fastest way to run each operator alone.
    best = best_unfused(k1, k2, inputs, R, BW, b_ser, b_k1, b_k2)
    best["batched_fused_over_best_unfused"] = round(b_f / best["batched_back_to_back_us"], 4)

    # fused forms the configuration names that are not the measured kernel, timed beside it
    extra = {}
    for label, a1, a2, akind, asuffix in BESIDE.get(number, []):
        if (a1, a2, akind, asuffix) == (k1, k2, kind, suffix):
            continue
        with bf.Operation(a1, a2) as op:
            op.upload(0, I1, F1)
            op.upload(1, I2, F2)
            alt = op.fused(akind, asuffix)
            op.zero_outputs()
            op.launch("serial")
            V1, V2 = op.download(0), op.download(1)
            op.zero_outputs()
            op.launch(akind, alt)
            Z1, Z2 = op.download(0), op.download(1)
            alt_exact = bool(np.array_equal(V1.view(np.uint8), Z1.view(np.uint8)) and np.array_equal(V2.view(np.uint8), Z2.view(np.uint8)))
            t_z = op.time(akind, alt, warmup=W, reps=R)[0]
            b_z = op.time_batched(akind, alt, warmup=BW, reps=R)
            b_zs = op.time_batched("serial", warmup=BW, reps=R)
        extra[label] = {"kernel": alt.name, "fused_us": round(float(t_z.mean()), 3), "batched_fused_us": round(b_z, 3),
                        "batched_back_to_back_us": round(b_zs, 3), "batched_fused_over_back_to_back": round(b_z / b_zs, 4),
                        "bit_exact_vs_unfused": alt_exact}
        bit_exact = bit_exact and alt_exact

    serial_sum = float(t_a.mean() + t_b.mean())
    back_to_back = float(t_ser.mean())
    if pair.bound == "mfma":
        achieved, unit = pair.flops / fused_us * 1e-6, "TFLOP/s"      # flops / us = MFLOP/s
        measured_peak = ceilings["mfma_bf16_TFLOPs" if pair.dtype == "bf16" else "mfma_f32_TFLOPs"]
    else:
        achieved, unit = (pair.bytes1 + pair.bytes2) / fused_us * 1e-3, "GB/s"
        measured_peak = ceilings["hbm_copy_GBps"]
    res = {
        "workload": f"pair {pair.number}: {pair.title}",
        "dtype": pair.dtype,
        "fused_kernel": fused.name, "grid": list(fused.grid), "block": list(fused.block),
        "fusion": note, "chooser": chooser,
        "bit_exact_vs_unfused": bit_exact,
        "fused_us": round(fused_us, 3),
        "fused_us_stats": {"min": round(float(t_f.min()), 3), "std": round(float(t_f.std()), 3),
                           "first_pass_mean": round(float(t_f1.mean()), 3)},
        "back_to_back_us": round(back_to_back, 3),
        "serial_sum_us": round(serial_sum, 3),
        "kernel1_us": round(float(t_a.mean()), 3),
        "kernel2_us": round(float(t_b.mean()), 3),
        "parallel_streams_us": round(float(t_par.mean()), 3),
        # first start -> second end includes the gap between the two launches (several us when each launch
        # waits for its own completion signal); the queued ratio below is the one quoted
        "fused_over_back_to_back_incl_launch_gap": round(fused_us / back_to_back, 4),
        "fused_over_serial_sum": round(fused_us / serial_sum, 4),
        "batched_fused_us": round(b_f, 3),
        "batched_back_to_back_us": round(b_ser, 3),
        "batched_kernel1_us": round(b_k1, 3),
        "batched_kernel2_us": round(b_k2, 3),
        "batched_fused_over_back_to_back": round(b_f / b_ser, 4),
        "fused_over_back_to_back": round(b_f / b_ser, 4),
        "best_unfused": best,
        "hip_graph": graph,
        "batched_rounds": {"fused_us": [round(x, 3) for x in q_f], "back_to_back_us": [round(x, 3) for x in q_ser]},
        "ms_per_step": round(wall_ms, 6),
        "baseline_reps": R,
        "roofline": {"bound": pair.bound, "achieved": round(achieved, 2), "peak": pair.peak, "unit": unit,
                     "frac": round(achieved / pair.peak, 4),
                     "measured_peak": measured_peak, "frac_of_measured_peak": round(achieved / measured_peak, 4),
                     "traffic": measured_traffic(fused.name),
                     "traffic_source": TRAFFIC_SOURCE.get(fused.name),
                     "kernel": fused.name, "avg_us": round(fused_us, 3),
                     "algorithmic": {"flops": pair.flops, "bytes": pair.bytes1 + pair.bytes2}},
        **extra,
    }
    if const:
        res["roofline"]["same_kernel_constant_operands"] = const
    if number in FLOORS:
        res["floor"] = FLOORS[number]
    return res, dev, inputs


def measure_group(name, K, W):
    """A fusion of more than two kernels (workloads.GROUPS): the fused kernel against its standalone
    kernels queued back to back, outputs compared byte for byte in the same run."""
    import bfuse_project_amd as bf
    from bfuse_project_amd import workloads as wl
    names, kind, suffixes, inputs = wl.GROUPS[name]
    with bf.GroupOperation(names) as op:
        for i, (I, F) in enumerate(inputs()):
            op.upload(i, I, F)
        op.zero_outputs()
        op.launch(op.unfused())
        want = [op.download(i) for i in range(len(names))]
        fused = op.fused(kind, suffixes[0])
        op.zero_outputs()
        op.launch([(fused, tuple(range(len(names))))])
        exact = all(np.array_equal(op.download(i).view(np.uint8), want[i].view(np.uint8)) for i in range(len(names)))
        R = max(K, BASELINE_MIN_REPS)
        each_u, queued_u = op.time(op.unfused(), warmup=max(W, R), reps=R)
        each_f, queued_f = op.time([(fused, tuple(range(len(names))))], warmup=max(W, R), reps=R)
    return {"kernels": list(names), "fused_kernel": fused.name, "fused_us": round(float(each_f[0]), 3),
            "kernel_us": [round(float(x), 3) for x in each_u], "batched_fused_us": round(queued_f, 3),
            "batched_back_to_back_us": round(queued_u, 3), "batched_fused_over_back_to_back": round(queued_f / queued_u, 4),
            "bit_exact_vs_unfused": bool(exact)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--pair", type=int, default=0, help="measure this pair only (default: all five, pair 5 on top)")
    ap.add_argument("--fusion", default="", help="'' = headline, 'auto' = the tuner's choice, or kind[:suffix][@k1,k2] with --pair")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-power-check", action="store_true",
                    help="skip the launches over constant operands (under a kernel trace they would be averaged into the fused kernel's figure)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures fused pairs on ONE GPU: the path has no cross-device data flow and "
                 "this build launches nothing on a second GPU; run with --gpus 1")
    if args.fusion not in ("", "auto") and not args.pair:
        sys.exit("--fusion kind[:suffix] pins a variant of one pair: give --pair N with it")

    K, W = args.steps, args.warmup
    numbers = [args.pair] if args.pair else [1, 2, 3, 4, 5]
    top = numbers[-1]
    pairs, top_inputs, dev = {}, None, ""
    ceilings = measured_ceilings()
    for n in numbers:
        res, dev, inputs = measure(n, K, W, args.fusion, ceilings, not args.no_power_check)
        pairs[str(n)] = res
        if n == top:
            top_inputs = inputs
    t = pairs[str(top)]
    out = {
        "metric": "fused-pair kernel us (speedup vs back-to-back launches; % roofline alongside)",
        "value": t["fused_us"],
        "unit": "us",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": t["ms_per_step"],
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": t["dtype"],
        "data": "synthetic (seeded, device-resident)",
        "config": {"workload": t["workload"], "fused_kernel": t["fused_kernel"], "grid": t["grid"], "block": t["block"],
                   "device": dev, "pairs_measured": numbers},
        "bit_exact_vs_unfused": all(p["bit_exact_vs_unfused"] for p in pairs.values()),
        "fused_over_back_to_back": t["fused_over_back_to_back"],
        "batched_fused_over_back_to_back": t["batched_fused_over_back_to_back"],
        "batched_fused_over_best_unfused": t["best_unfused"]["batched_fused_over_best_unfused"],
        "roofline": t["roofline"],
        "hbm_copy_GBps": ceilings["hbm_copy_GBps"],
        "measured_ceilings": ceilings,
        "pairs": pairs,
    }
    # the stated target: every fused pair of configurations 1-4 in at most 0.9 x the time of the same two
    # kernels launched back to back (queued: the strongest form of that baseline)
    tgt = {n: pairs[n]["batched_fused_over_back_to_back"] for n in ("1", "2", "3", "4") if n in pairs}
    if tgt:
        # the same target against the fastest standalone kernels the library holds for each operator
        # (not always the ones the fused kernel was built from): stated beside it
        vs_best = {n: pairs[n]["best_unfused"]["batched_fused_over_best_unfused"] for n in tgt}
        out["target"] = {"queued_fused_over_back_to_back_at_most": 0.9, "pairs": tgt, "met": all(v <= 0.9 for v in tgt.values()),
                         "pairs_vs_best_unfused": vs_best, "met_vs_best_unfused": all(v <= 0.9 for v in vs_best.values())}
    if not args.pair:
        from bfuse_project_amd.workloads import GROUPS
        out["groups"] = {g: measure_group(g, K, W) for g in GROUPS}
        out["bit_exact_vs_unfused"] = out["bit_exact_vs_unfused"] and all(g["bit_exact_vs_unfused"] for g in out["groups"].values())
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(top, *top_inputs)
    print(json.dumps(out))
    if not out["bit_exact_vs_unfused"]:
        sys.exit("a fused kernel's output differs from the unfused kernels")


if __name__ == "__main__":
    main()
