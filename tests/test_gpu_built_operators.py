"""Operators built after the library for a user config (configure --build-missing / build_operators): the reference
generates a kernel for whatever arguments an operator id has (scripts/configure_kernels.py:40-69); here an id of a
shape the library lacks is an instantiation of one of its templates at the default tiling, compiled into a module
of the suite.

The suite is bfuse-project_amd/examples/new_shapes.yaml, configured and built in-tree by the build step: six
operators of new shapes (3 x 3 and 1 x 1 convolutions of small batches, a 5 x 5 / stride 2 on RGB, two batched
products -- one of 100 x 72 matrices that no tile divides --, a dense layer with its weight in the reference's (out, in) layout) and one the library holds.  Every
built operator against the CPU oracle at full size (1e-5 of max(|ref|, rms)); every fused kernel of the
suite's pairs bit for bit against the two kernels back to back; the suite and the command-line driver over it."""
import os
import subprocess

import numpy as np
import pytest
import yaml

import bfuse_project_amd as bf
from bfuse_project_amd import build_pairs, suite
from bfuse_project_amd.operation import fill_normal
from oracle import oracle as orf
from tests import oracle_cases

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SUITE = os.path.join(ROOT, "bfuse-project_amd", "examples", "built", "new_shapes")
BENCH = os.path.join(ROOT, "bfuse-project_amd", "benchmark")
PARTNER = "layernorm_512x768"


@pytest.fixture(scope="module")
def built():
    assert os.path.exists(os.path.join(SUITE, "config", "modules.yaml")), \
        "the sample suite has not been built: python -c 'import __graft_entry__ as g; g.build()'"
    modules = build_pairs.load_suite_modules(SUITE)
    assert len(modules) == 2 and modules[0].endswith(os.path.join("hip", "operators", "libbfuse_pairs.so"))
    with open(os.path.join(SUITE, "config", "info.yaml")) as f:
        info = yaml.safe_load(f)
    return modules, info


def _oracle(kid, args, I, F):
    if kid.startswith("conv2d"):
        n, h, w, co, ci, kh, kw, s, p = args
        return orf.conv2d(I.reshape(n, ci, h, w), F.reshape(co, ci, kh, kw), s=s, p=p)
    if kid.startswith("bgemm"):
        b, m, k, n = args
        return np.stack([orf.gemm_f32(I.reshape(b, m, k)[x], F.reshape(b, n, k)[x], b_is_nk=True) for x in range(b)])
    b, i, o = args
    return orf.gemm_f32(I.reshape(b, i), F.reshape(o, i), b_is_nk=True)     # the weight as the reference stores it: (out, in)


def test_every_built_operator_against_the_oracle(built):
    _, info = built
    checked = 0
    for kid, d in info["Resolved"].items():
        args = info["KernelInfo"][kid]
        if d["kernel"] == "gemm_f32_512x768x768":      # the one id the library holds
            continue
        name = d["kernel"]
        print(f"[built-op] {kid} {args} -> {name}", flush=True)
        with bf.Operation(name, PARTNER) as op:
            k = op.k[0]
            I = fill_normal(0x0B0 + checked, int(np.prod(k.shapes[0])), 0.0, 1.0)
            F = fill_normal(0x0C0 + checked, int(np.prod(k.shapes[1])), 0.0, 0.1)
            got = op.run_kernel(0, I, F)
        want = _oracle(kid, args, I, F)
        assert got.size == want.size
        st = oracle_cases.rel_stats(got.reshape(want.shape), want, 1e-5)
        print(f"[parity] {name}: worst |d|/max(|ref|,rms) {st['worst_floor_rel']:.3e}; {st['n_fail']} fail", flush=True)
        assert st["n_fail"] == 0
        checked += 1
    assert checked == 6
    assert info["Resolved"]["dense_0"] == {"kernel": "gemm_f32_48x160x96_nk", "dtype": "f32", "weight_layout": "reference", "weight_transpose": None}


def test_fused_kernels_of_built_operators_equal_the_two_kernels_back_to_back(built):
    _, info = built
    a, b = suite.set_names(info)
    n = 0
    for i, k1 in enumerate(a):
        for j, k2 in enumerate(b):
            variants = suite.fused_variants(k1, k2)
            assert variants["bfuse"], f"{k1} + {k2}: no block-fused kernel in the module"
            print(f"[built-op] {k1} + {k2}: {[f.name for f in variants['bfuse'] + variants['hfuse']]}", flush=True)
            with bf.Operation(k1, k2) as op:
                I1, F1 = suite._synthetic(op.k[0], 0xD0 + 2 * i)
                I2, F2 = suite._synthetic(op.k[1], 0xE0 + 2 * j)
                want = (op.run_kernel(0, I1, F1), op.run_kernel(1, I2, F2))
                for kind in ("bfuse", "hfuse"):
                    for f in variants[kind]:
                        q1, q2 = op.run_fuse(f, I1, F1, I2, F2)
                        assert q1.tobytes() == want[0].tobytes() and q2.tobytes() == want[1].tobytes(), f"{f.name}: output differs from the unfused kernels"
                        n += 1
    assert n >= 12


def test_suite_and_driver_run_over_built_operators(built, tmp_path):
    modules, info = built
    rows = suite.run_suite(info, str(tmp_path), validate=True, log=lambda *a: None)
    assert len(rows) == 12 and all(r["serial_ns"] > 0 for r in rows)
    info_path = os.path.join(SUITE, "config", "info.yaml")
    env = dict(os.environ, BFUSE_KERNEL_MODULES=":".join(modules))
    # conv2d_1 (index 1 of set 0) with bgemm_1 (index 1 of set 1): both built operators, block-fused, validated
    r = subprocess.run([BENCH, "-v", "-n", "1", "-i", info_path, "-x", "_c256", "4", "1", "1"], env=env, capture_output=True, text=True, timeout=300)
    print(r.stdout[-600:], r.stderr[-300:], flush=True)
    assert r.returncode == 0 and "INVALID" not in r.stdout and r.stdout.count("VALID") >= 2
    r = subprocess.run([BENCH, "-n", "1", "-i", info_path, "0", "1", "1"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0, "without the modules the driver has no such kernel"
