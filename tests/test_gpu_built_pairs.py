"""Fused kernels built after the library for a configured suite (build_pairs): the reference generates and
compiles the fused kernels of every pair of a user's config (scripts/configure_kernels.py:229-320,
scripts/quick_start.py:44-55); here the pairs the library holds no fused kernel for are written as
instantiations over the registered operators and compiled into a module of their own.

The suite is bfuse-project_amd/examples/batch_operators.yaml (four batch-1024 operators of the reference's
benchmark.yaml / inception_v3.yaml), configured and built in-tree by the build step.  Every fused kernel of
its module must write what the two kernels write back to back, bit for bit, over all 1024 items -- compared
through device-side checksums of every item and a downloaded sample; the command-line driver must find the
module through BFUSE_KERNEL_MODULES and validate a pair; the suite must run over it."""
import os
import subprocess

import numpy as np
import pytest
import yaml

import bfuse_project_amd as bf
from bfuse_project_amd import build_pairs, suite
from tests import perf_report

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SUITE = os.path.join(ROOT, "bfuse-project_amd", "examples", "built", "batch_operators")
BENCH = os.path.join(ROOT, "bfuse-project_amd", "benchmark")


@pytest.fixture(scope="module")
def modules():
    assert os.path.exists(os.path.join(SUITE, "config", "modules.yaml")), \
        "the sample suite has not been built: python -c 'import __graft_entry__ as g; g.build()'"
    return build_pairs.load_suite_modules(SUITE)


def _items(op, side):
    """Per-item checksums of a side's output (1024 items) and its first and last items."""
    total = int(np.prod(op.k[side].shapes[2]))
    item = total // 1024
    return op.checksum_output(side, item), op.download_part(side, 0, 2 * item), op.download_part(side, total - 2 * item, 2 * item)


def test_every_built_pair_equals_the_two_kernels_back_to_back(modules):
    info = suite.load_info(os.path.join(SUITE, "config", "info.yaml"))
    a, b = suite.set_names(info)
    built = 0
    for i, k1 in enumerate(a):
        for j, k2 in enumerate(b):
            variants = suite.fused_variants(k1, k2)
            assert variants["bfuse"], f"{k1} + {k2}: no block-fused kernel in the module"
            with bf.Operation(k1, k2) as op:
                I1, F1 = suite._synthetic(op.k[0], 0xB0 + 2 * i)
                I2, F2 = suite._synthetic(op.k[1], 0xC0 + 2 * j)
                op.upload(0, I1, F1)
                op.upload(1, I2, F2)
                op.zero_outputs()
                op.launch("serial")
                want = [_items(op, s) for s in (0, 1)]
                assert all(w[0][:, 0].any() for w in want), "an unfused kernel wrote nothing"
                t_ser = op.time_batched("serial", warmup=2, reps=5)
                for kind in ("bfuse", "hfuse"):
                    for f in variants[kind]:
                        op.zero_outputs()
                        op.launch(kind, f)
                        for s in (0, 1):
                            got = _items(op, s)
                            bad = np.flatnonzero((got[0] != want[s][0]).any(axis=1))
                            assert bad.size == 0, f"{f.name}: side {s}: {bad.size} of 1024 items differ, first {bad[:8]}"
                            assert got[1].tobytes() == want[s][1].tobytes() and got[2].tobytes() == want[s][2].tobytes()
                        t = op.time_batched(kind, f, warmup=2, reps=5)
                        print(f"[built] {f.name}: {t:.0f} us fused, {t_ser:.0f} us back to back ({t / t_ser:.3f})", flush=True)
                        built += 1
    assert built >= 6


def test_driver_finds_the_module_through_the_environment(modules):
    info_path = os.path.join(SUITE, "config", "info.yaml")
    env = dict(os.environ, BFUSE_KERNEL_MODULES=":".join(modules))
    # conv2d1_25 (index 1 of set 0) with bgemm2_8 (index 0 of set 1), block-fused, validated against the unfused kernels
    r = subprocess.run([BENCH, "-v", "-n", "1", "-i", info_path, "-x", "_c256", "4", "1", "0"], env=env, capture_output=True, text=True, timeout=300)
    print(r.stdout[-600:], r.stderr[-600:], flush=True)
    assert r.returncode == 0, r.stderr
    # the same through the driver's resident mode: operands written and outputs compared on the device
    r = subprocess.run([BENCH, "-v", "-r", "-n", "3", "-i", info_path, "-x", "_c256", "4", "1", "0"], env=env, capture_output=True, text=True, timeout=300)
    print(r.stdout[-600:], r.stderr[-600:], flush=True)
    assert r.returncode == 0 and r.stdout.count("VALID (checksums") == 2 and "INVALID" not in r.stdout, r.stdout + r.stderr
    r = subprocess.run([BENCH, "-v", "-r", "-n", "3", "-i", info_path, "3", "1", "0"], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "INVALID" not in r.stdout, r.stdout + r.stderr          # thread-level fusion of the same pair
    # without the module the same command has no fused kernel to run
    r = subprocess.run([BENCH, "-d", "-i", info_path, "-x", "_c256", "4", "1", "0"], env={k: v for k, v in os.environ.items() if k != "BFUSE_KERNEL_MODULES"},
                       capture_output=True, text=True, timeout=60)
    assert r.returncode != 0


def test_suite_runs_the_built_pairs(modules, tmp_path):
    info = suite.load_info(os.path.join(SUITE, "config", "info.yaml"))
    rows = suite.run_suite(info, str(tmp_path), validate=True, log=lambda *a: None)
    assert len(rows) == 4
    for r in rows:
        assert r["chooser"]["kind"] in ("bfuse", "hfuse", "none")
        assert "bfuse_ns" in r, "the block-fused kernel of the module was not run"
        print(f"[built] {r['kernel1']} + {r['kernel2']}: chooser {r['chooser']['kind']}, {r['chooser_speedup']:.3f}x of the two kernels one after the other; "
              f"block-fused {r['bfuse_speedup']:.3f}x" + (f", thread-fused {r['hfuse_speedup']:.3f}x" if "hfuse_speedup" in r else ""), flush=True)
    perf_report.expect(all(r["chooser_speedup"] >= 0.97 for r in rows), "the chooser's form is not slower than the two kernels one after the other")


def test_resident_suite_run_and_device_fill(modules, tmp_path):
    """The suite's mode for operators of several GB: operands written on the device must be the operands the
    host fill gives (the same kernel over both gives the same output, bit for bit), and the run -- fused outputs
    compared with the unfused ones through device-side checksums -- must come out like the host-side one."""
    from bfuse_project_amd.operation import fill_uniform
    k1, k2 = "bgemm_f32_1024x208x64x208", "gemm_f32_1024x768x768"
    with bf.Operation(k1, k2) as op:
        outs = []
        for how in ("host", "device"):
            for side in (0, 1):
                n = [int(np.prod(op.k[side].shapes[t])) for t in (0, 1)]
                if how == "host":
                    op.upload(side, fill_uniform(77 + side, n[0], -0.5, 0.5), fill_uniform(177 + side, n[1], -0.5, 0.5))
                else:
                    op.upload(side, np.zeros(n[0], np.float32), np.zeros(n[1], np.float32))
                    op.fill_uniform_device(side, 0, 77 + side, -0.5, 0.5)
                    op.fill_uniform_device(side, 1, 177 + side, -0.5, 0.5)
            op.zero_outputs()
            op.launch("serial")
            outs.append((op.download(0), op.download(1)))
        assert outs[0][0].any() and outs[0][0].tobytes() == outs[1][0].tobytes() and outs[0][1].tobytes() == outs[1][1].tobytes()
    info = suite.load_info(os.path.join(SUITE, "config", "info.yaml"))
    rows = suite.run_suite(info, str(tmp_path), validate=True, log=lambda *a: None, resident=True, rows=(1, 2))
    assert len(rows) == 2 and all("bfuse_ns" in r for r in rows)           # the pairs of the second operator of set 0
    for r in rows:
        # two matrix-core kernels that each cover the chip: left unfused
        assert r["chooser"]["kind"] == "none" and r["chooser_speedup"] == 1.0


def test_tuner_times_plans_on_a_built_run_time_plan_kernel(modules):
    """build_pairs --rt: the pair's block-fused kernel with its dispatch plan as run-time data.  Every candidate
    plan and persistent workgroup count must leave both outputs what the unfused kernels write (checksums of
    all 1024 items), and the tuner ranks them."""
    from bfuse_project_amd import patterns, tuner
    k1, k2 = "conv1x1s1p0_f32_1024x1280x8x8_192", "bgemm_f32_1024x208x64x208"
    with bf.Operation(k1, k2) as op:
        for side in (0, 1):
            op.fill_uniform_device(side, 0, 31 + side, -0.5, 0.5)
            op.fill_uniform_device(side, 1, 41 + side, -0.5, 0.5)
        op.zero_outputs()
        op.launch("serial")
        want = [op.checksum_output(s, int(np.prod(op.k[s].shapes[2])) // 1024) for s in (0, 1)]
        rt = op.fused_rt()
        dims = [patterns.LaunchDims(tuple(k.grid), tuple(k.block)) for k in op.k]
        cands = [tuner.Candidate("ranges", "ranges"), tuner.Candidate("chunk 256", "chunked", 256), tuner.Candidate("zigzag 1:1", "zigzag", 1, 1),
                 tuner.Candidate("chunk 256, 1024 persistent workgroups", "chunked", 256, 1, 1024)]
        for c in cands:
            h = op.set_plan(rt, patterns.plan_blocks(c.pattern, dims, c.p0, c.p1), c.workgroups)
            op.zero_outputs()
            op.launch("bfuse", h)
            for s in (0, 1):
                got = op.checksum_output(s, int(np.prod(op.k[s].shapes[2])) // 1024)
                assert np.array_equal(got, want[s]), f"{c.label}: side {s} differs from the unfused kernel"
        rows = tuner.autotune(op, cands, warmup=2, reps=5)
        for r in rows:
            print(f"[built] {k1} + {k2}: {r['label']:42s} {r['us_mean']:.0f} us", flush=True)
        assert len(rows) == len(cands) and rows[0]["us_mean"] <= rows[-1]["us_mean"]
