"""Fusions of three and four kernels on the MI355X, through the C ABI's launch lists: every fused
output must equal the unfused one bit for bit, and the unfused outputs are within tolerance of the
CPU oracle.  Small groups cover every block pattern, the run-time plans with persistent workgroups
and the thread-level forms; one full-size group (QKV projection, LayerNorm, causal softmax) is also
timed against its three kernels queued back to back.
"""
import sys

import numpy as np
import pytest

import bfuse_project_amd as bf
from bfuse_project_amd import patterns, tuner
from bfuse_project_amd.workloads import GROUPS as WORKLOAD_GROUPS
from tests import oracle_cases
from tests.perf_report import expect
from tests.test_gpu_small import _cases, _check
from tests.test_group_host import GROUPS

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _same(a, b):
    return bool(np.array_equal(np.ascontiguousarray(a).view(np.uint8).ravel(), np.ascontiguousarray(b).view(np.uint8).ravel()))


SMALL = [g for g in GROUPS if not g[0][0].startswith("gemm_f32_512")]


@pytest.mark.parametrize("names,kind,suffix,pattern", SMALL)
def test_small_groups_bit_exact_and_close_to_cpu(names, kind, suffix, pattern):
    cases = _cases()
    ins = [cases[n][0](300 + 11 * i) for i, n in enumerate(names)]
    _say(f"[group] {' + '.join(names)} {kind}{suffix}")
    with bf.GroupOperation(names) as op:
        for i, (I, F) in enumerate(ins):
            op.upload(i, I, F)
        op.zero_outputs()
        op.launch(op.unfused())
        want = [op.download(i) for i in range(len(names))]
        fused = op.fused(kind, suffix)
        outs = []
        for rep in range(2):   # a second launch over the same buffers gives the same bytes
            op.zero_outputs()
            op.launch([(fused, tuple(range(len(names))))])
            outs.append([op.download(i) for i in range(len(names))])
    for i, n in enumerate(names):
        assert _same(outs[0][i], want[i]) and _same(outs[1][i], want[i]), f"{n}: fused output differs from the standalone kernel's"
        e = _check(n, want[i], cases[n][1](*ins[i]), cases[n][2], cases[n][3])
        _say(f"[group]   {n}: bit-exact, max rel err vs CPU {e:.3e}")


def test_run_time_plans_over_three_kernels_with_persistent_workgroups():
    names = ("conv3x3_f32_32x12x12_32", "gemm_gelu_f32_96x128x192", "bias_relu_4096")
    cases = _cases()
    ins = [cases[n][0](500 + 7 * i) for i, n in enumerate(names)]
    with bf.GroupOperation(names) as op:
        for i, (I, F) in enumerate(ins):
            op.upload(i, I, F)
        op.launch(op.unfused())
        want = [op.download(i) for i in range(3)]
        rt = op.fused("bfuse", "_rt")
        dims = [bf.LaunchDims(k.grid, k.block) for k in op.k]
        total = sum(k.grid[0] for k in op.k)
        for pattern, params in (("zigzag", (1, 1)), ("zigzag", (2, 1)), ("proportional", (3, 1)), ("chunked", (4, 1)), ("ranges", ())):
            plan = bf.plan_blocks(pattern, dims, *params)
            for wgs in (None, 1, 3, total // 2, total - 1):
                _say(f"[group-rt] {pattern} {params} workgroups={wgs}")
                h = op.set_plan(rt, plan, wgs)
                op.zero_outputs()
                op.launch([(h, (0, 1, 2))])
                for i in range(3):
                    assert _same(op.download(i), want[i]), (pattern, params, wgs, names[i])
        # a plan over two grids is not a plan of this kernel
        with pytest.raises(bf.BfuseError):
            op.set_plan(rt, bf.plan_blocks("ranges", dims[:2]))


def test_launch_lists_check_their_arguments():
    names = ("conv3x3_f32_32x12x12_32", "gemm_gelu_f32_96x128x192", "bias_relu_4096")
    with bf.GroupOperation(names) as op:
        fused = op.fused("bfuse", "_r")
        with pytest.raises(bf.BfuseError, match="3 sides"):
            op.launch([(fused, (0, 1))])
        with pytest.raises(bf.BfuseError, match="named twice"):
            op.launch([(fused, (0, 1, 1))])
        with pytest.raises(bf.BfuseError):            # side 4 was never initialised
            op.launch([(fused, (0, 1, 3))])
        with pytest.raises(bf.BfuseError):            # the buffers of side 3 are too small for the GEMM
            op.launch([(fused, (2, 1, 0))])
        with pytest.raises(bf.BfuseError):            # wrong launch shape
            op.launch([(bf.operation.replace(fused, grid=(fused.grid[0] + 1, 1, 1)), (0, 1, 2))])
        # a pair kernel of the library runs over any two sides that fit it
        pair = bf.kernel_info("conv3x3_f32_32x12x12_32_gemm_gelu_f32_96x128x192_fused_bfuse_c4")
        cases = _cases()
        ins = [cases[n][0](40 + i) for i, n in enumerate(names)]
        for i, (I, F) in enumerate(ins):
            op.upload(i, I, F)
        op.launch(op.unfused())
        want = [op.download(i) for i in range(3)]
        op.zero_outputs()
        op.launch([(pair, (0, 1)), (op.k[2], (2,))])
        for i in range(3):
            assert _same(op.download(i), want[i])
    # the two-sided harness refuses a kernel of three
    with bf.Operation(names[0], names[1]) as op2:
        with pytest.raises(bf.BfuseError, match="9 pointers"):
            op2.launch("bfuse", fused)


def test_full_size_three_kernels_bit_exact_close_to_cpu_and_timed():
    names, _, _, inputs = WORKLOAD_GROUPS["qkv_ln_softmax"]
    (I1, F1), (I2, F2), (I3, F3) = inputs()
    E1, E2 = oracle_cases.expected(2, I1, F1, I2, F2)
    from oracle import oracle as orf
    E3 = orf.softmax_causal(np.asarray(I3).reshape(12, 512, 512))
    with bf.GroupOperation(names) as op:
        for i, (I, F) in enumerate(((I1, F1), (I2, F2), (I3, F3))):
            op.upload(i, I, F)
        op.launch(op.unfused())
        want = [op.download(i) for i in range(3)]
        for got, exp, n in zip(want, (E1, E2, E3), names):
            e = oracle_cases.rel_error(np.asarray(got).ravel(), np.asarray(exp).ravel())
            _say(f"[group-full] {n}: max rel err vs CPU {e:.3e}")
            assert e <= 1e-5
        each_u, queued_u = op.time(op.unfused(), warmup=20, reps=300)
        for suffix in ("_r", "_c256"):
            fused = op.fused("bfuse", suffix)
            op.zero_outputs()
            op.launch([(fused, (0, 1, 2))])
            for i in range(3):
                assert _same(op.download(i), want[i]), (suffix, names[i])
            each_f, queued_f = op.time([(fused, (0, 1, 2))], warmup=20, reps=300)
            _say(f"[group-full] bfuse{suffix}: fused {each_f[0]:.2f} us (queued {queued_f:.2f}); unfused {' + '.join(f'{x:.2f}' for x in each_u)} = "
                 f"{each_u.sum():.2f} us (queued {queued_u:.2f}); queued fused / unfused = {queued_f / queued_u:.3f}")
        rt = op.fused("bfuse", "_rt")
        dims = [bf.LaunchDims(k.grid, k.block) for k in op.k]
        h = op.set_plan(rt, bf.plan_blocks("ranges", dims))
        op.zero_outputs()
        op.launch([(h, (0, 1, 2))])
        for i in range(3):
            assert _same(op.download(i), want[i]), ("rt", names[i])
        # three kernels hidden behind one: the fused kernel beats the queued triple clearly (reported, not asserted)
        expect(queued_f < 0.95 * queued_u, f"group of three queued: fused {queued_f:.2f} us, unfused {queued_u:.2f} us")


def test_autotune_of_the_full_size_group_agrees_with_the_footprint_rule():
    """Candidate plans timed on the group's run-time-plan kernel: the rule's plan (one chunk per round
    over the CUs) is reported against the best candidate with one workgroup per fused block, and
    the compile-time kernel with that dispatch is the one the benchmark measures."""
    names, kind, suffixes, inputs = WORKLOAD_GROUPS["qkv_ln_softmax"]
    with bf.GroupOperation(names) as op:
        for i, (I, F) in enumerate(inputs()):
            op.upload(i, I, F)
        op.launch(op.unfused())
        want_out = [op.download(i) for i in range(len(names))]
        choice = tuner.static_plan_group(op.k)
        dims = [patterns.LaunchDims(tuple(k.grid), tuple(k.block)) for k in op.k]
        want = patterns.plan_blocks(choice["pattern"], dims, choice["p0"], choice["p1"])

        def timed():
            rows = tuner.autotune_group(op, warmup=20, reps=100)
            plain = [r for r in rows if not r["persistent"]]
            mine = [r for r in plain if tuner.same_dispatch(want, patterns.plan_blocks(r["pattern"], dims, r["p0"], r["p1"]))]
            return rows, mine, min(r["us_mean"] for r in plain)

        rows, mine, best_plain = timed()
        for r in rows:
            _say(f"[tune-group] {r['label']:44s} {r['us_mean']:8.2f} us (queued {r['us_queued']:.2f}) workgroups {r['workgroups']}")
        assert mine, "the footprint rule's plan is not among the candidates"
        _say(f"[tune-group] footprint rule -> {mine[0]['label']} {mine[0]['us_mean']:.2f} us, best plain candidate {best_plain:.2f} us")
        expect(min(r["us_mean"] for r in mine) <= 1.03 * best_plain,
               f"group: the footprint rule's plan {min(r['us_mean'] for r in mine):.2f} us, best plain candidate {best_plain:.2f} us")
        # the winner, installed again, still reproduces the standalone kernels
        best = rows[0]
        h = op.set_plan(op.fused("bfuse", "_rt"), patterns.plan_blocks(best["pattern"], dims, best["p0"], best["p1"]), best["workgroups"])
        op.zero_outputs()
        op.launch([(h, tuple(range(len(names))))])
        for i in range(len(names)):
            assert _same(op.download(i), want_out[i]), (best["label"], names[i])
        v = tuner.find_group_variant(op.k, choice)
        assert v is not None and v.name == "_".join(names) + f"_fused_{kind}{suffixes[0]}"
