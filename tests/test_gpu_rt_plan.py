"""Block fusion with the dispatch plan as run-time data, and persistent workgroups.

`<K1>_<K2>_fused_bfuse_rt` kernels take their BlockPlan from device memory (bfuse_set_plan) and
stride over the fused block ids, so one compiled kernel serves every pattern / ratio / grid.
Whatever the plan and the number of workgroups, each side must produce the bytes of its
standalone kernel.  The tuner (bfuse_project_amd.tuner) is the run-time form of the reference's
ratio sweep (legacy/tests/single_bgemm_conv2d/auto.py:9-30).
"""
import ctypes as C

import numpy as np
import pytest

import bfuse_project_amd as bf
from bfuse_project_amd import patterns, tuner
from bfuse_project_amd._lib import BfuseError
from bfuse_project_amd.workloads import CONFIG_KINDS, HEADLINE, PAIRS, RT_SIDES
from tests.perf_report import expect
from tests.test_gpu_small import _cases

pytestmark = pytest.mark.gpu

SMALL = [
    ("gemm_f32_128x160x192_d", "bias_relu_4096"),                 # split-K GEMM (epilogue barriers) + barrier-free side
    ("conv3x3_f32_32x12x12_32", "gemm_gelu_f32_96x128x192"),      # both sides end in a barrier
    ("layernorm_8x256", "softmax_causal_2x256x256"),
    ("gemm_bf16_256x320x1792_w8", "rmsnorm_rope_bf16_6x1024"),    # fence-free barriers of the direct-to-LDS GEMM
]
PLANS = [("zigzag", 1, 1), ("zigzag", 2, 3), ("zigzag", 8, 1), ("chunked", 4, 1), ("chunked", 256, 1), ("proportional", 1, 1), ("ranges", 1, 1)]


def test_launch_without_a_plan_is_refused():
    k1, k2 = SMALL[0]
    with bf.Operation(k1, k2) as op:
        rt = op.fused_rt()
        assert rt.kind == 3
        with pytest.raises(BfuseError, match="no plan"):
            op.launch("bfuse", rt)


@pytest.mark.parametrize("k1,k2", SMALL)
def test_every_plan_and_grid_reproduces_the_unfused_kernels(k1, k2):
    cases = _cases()
    I1, F1 = cases[k1][0](31)
    I2, F2 = cases[k2][0](47)
    with bf.Operation(k1, k2) as op:
        O1, O2 = op.run_kernel(0, I1, F1), op.run_kernel(1, I2, F2)
        rt = op.fused_rt()
        dims = [patterns.LaunchDims(tuple(k.grid), tuple(k.block)) for k in op.k]
        total = op.k[0].grid[0] + op.k[1].grid[0]
        for pattern, p0, p1 in PLANS:
            plan = patterns.plan_blocks(pattern, dims, p0, p1)
            assert plan.fused_grid == total
            for wgs in (None, 1, 3, max(1, total // 2), total - 1):
                h = op.set_plan(rt, plan, wgs)
                print(f"[rt] {rt.name} {pattern} {p0}:{p1} workgroups {h.grid[0]}", flush=True)
                op.zero_outputs()
                Q1, Q2 = op.run_fuse(h, I1, F1, I2, F2)
                assert np.array_equal(Q1.view(np.uint8), O1.view(np.uint8)), (pattern, p0, p1, wgs, k1)
                assert np.array_equal(Q2.view(np.uint8), O2.view(np.uint8)), (pattern, p0, p1, wgs, k2)


def test_bad_plans_and_grids_are_refused():
    k1, k2 = SMALL[2]
    with bf.Operation(k1, k2) as op:
        rt = op.fused_rt()
        dims = [patterns.LaunchDims(tuple(k.grid), tuple(k.block)) for k in op.k]
        good = patterns.plan_blocks("zigzag", dims, 1, 1)
        # a plan made for other grids
        other = patterns.plan_blocks("zigzag", [patterns.LaunchDims((dims[0].grid[0] + 1, 1, 1), dims[0].block), dims[1]], 1, 1)
        with pytest.raises(BfuseError, match="covers"):
            op.set_plan(rt, other)
        # a plan that sends two fused blocks to the same virtual block
        bent = patterns.plan_blocks("ranges", dims, 1, 1)
        bent.c.seg[bent.c.n_seg - 1].slot[0].base += 1
        with pytest.raises(BfuseError, match="out of range or visited twice"):
            op.set_plan(rt, bent)
        bent = patterns.plan_blocks("ranges", dims, 1, 1)
        bent.c.seg[0].period = 0
        with pytest.raises(BfuseError, match="malformed"):
            op.set_plan(rt, bent)
        # not a run-time-plan kernel
        with pytest.raises(BfuseError, match="not a run-time-plan"):
            op.set_plan(op.fused("bfuse"), good)
        h = op.set_plan(rt, good)
        from dataclasses import replace
        with pytest.raises(BfuseError, match="1-D grid"):
            op.launch("bfuse", replace(h, grid=(good.fused_grid + 1, 1, 1)))
        with pytest.raises(BfuseError, match="block"):
            op.launch("bfuse", replace(h, block=(64, 1, 1)))


def test_pair1_footprint_selects_thread_level_fusion():
    """Pair 1's configuration is thread-level fusion; with the real register and LDS figures the
    footprint rule selects it unprompted (matching grids, one barrier-free side, LDS and threads fit)."""
    k1, k2 = RT_SIDES[1]
    with bf.Operation(k1, k2) as op:
        st = tuner.static_choice(op.k[0], op.k[1])
        print(f"[tune] pair 1 static: {st}  regs {op.k[0].regs}/{op.k[1].regs} lds {op.k[0].lds_bytes}/{op.k[1].lds_bytes}", flush=True)
        assert op.k[0].regs > 0 and op.k[0].lds_bytes > 0          # metadata comes from the code object
        assert st["hfuse_ok"] and st["prefer"] == "hfuse"
        h = tuner.find_variant(op.k[0], op.k[1], tuner.static_plan(op.k[0], op.k[1], kinds=CONFIG_KINDS[1]))
        assert h is not None and h.name == op.fused("hfuse").name


@pytest.mark.parametrize("number", [2, 3, 4, 5])
def test_autotune_full_size_agrees_with_the_footprint_rule_and_the_headline(number):
    """Times the candidate plans on the pair's run-time-plan kernel.  The plan the footprint rule
    selects (the headline kernel's dispatch) is reported against the best candidate that has
    one workgroup per fused block; times are printed, not asserted (persistent-workgroup launches exist only on the run-time-plan
    kernel, so they cannot be the compile-time headline)."""
    pair = PAIRS[number]
    k1, k2 = RT_SIDES[number]
    hk1, hk2, hkind, hsuffix = HEADLINE[number]
    I1, F1, I2, F2 = pair.inputs()
    with bf.Operation(k1, k2) as op:
        O1, O2 = op.run_kernel(0, I1, F1), op.run_kernel(1, I2, F2)
        op.upload(0, I1, F1)
        op.upload(1, I2, F2)
        choice = tuner.static_plan(op.k[0], op.k[1], kinds=CONFIG_KINDS[number])
        rows = tuner.autotune(op, warmup=20, reps=100)
        assert rows == sorted(rows, key=lambda r: r["us_mean"]) and rows[0]["us_mean"] > 0
        print(f"[tune] pair {number} static: {choice}")
        for r in rows:
            print(f"[tune] pair {number}: {r['label']:44s} {r['us_mean']:8.2f} us (median {r['us_median']:.2f}, min {r['us_min']:.2f}) workgroups {r['workgroups']}", flush=True)
        # the winner, installed again, still reproduces the unfused kernels
        best = rows[0]
        dims = [patterns.LaunchDims(tuple(k.grid), tuple(k.block)) for k in op.k]
        h = op.set_plan(op.fused_rt(), patterns.plan_blocks(best["pattern"], dims, best["p0"], best["p1"]), best["workgroups"])
        op.zero_outputs()
        Q1, Q2 = op.run_fuse(h, I1, F1, I2, F2)
        assert np.array_equal(Q1.view(np.uint8), O1.view(np.uint8)) and np.array_equal(Q2.view(np.uint8), O2.view(np.uint8))
        # the footprint rule's plan among the timed candidates
        assert choice["kind"] == "bfuse"
        want = patterns.plan_blocks(choice["pattern"], dims, choice["p0"], choice["p1"])
        plain = [r for r in rows if not r["persistent"]]
        mine = [r for r in plain if tuner.same_dispatch(want, patterns.plan_blocks(r["pattern"], dims, r["p0"], r["p1"]))]
        assert mine, "the footprint rule's plan is not among the candidates"
        best_plain = min(r["us_median"] for r in plain)
        print(f"[tune] pair {number}: footprint rule -> {mine[0]['label']} {mine[0]['us_median']:.2f} us, best plain candidate {best_plain:.2f} us", flush=True)
        expect(min(r["us_median"] for r in mine) <= 1.03 * best_plain,
               f"pair {number}: the footprint rule's plan {min(r['us_median'] for r in mine):.2f} us, best plain candidate {best_plain:.2f} us")
        # the 1:1 zig-zag (the reference's live pattern) is not the best placement on this chip
        zz = [r for r in rows if r["label"] == "zigzag 1:1"][0]
        expect(rows[0]["us_mean"] <= zz["us_mean"], f"pair {number}: best plan {rows[0]['us_mean']:.2f} us, 1:1 zig-zag {zz['us_mean']:.2f} us")
    # and the compile-time kernel with that dispatch is the headline kernel
    a, b = bf.kernel_info(hk1), bf.kernel_info(hk2)
    v = tuner.find_variant(a, b, tuner.static_plan(a, b, kinds=CONFIG_KINDS[number]))
    assert v is not None and v.name == f"{hk1}_{hk2}_fused_{hkind}{hsuffix}"
