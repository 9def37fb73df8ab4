"""Kernels emitted by the front end, run on the GPU.

`tests/frontend/Makefile` ran `horizontal-fuser` over tests/frontend/kernels.cu and compiled
its outputs to gfx950 code objects ahead of time.  Each fused kernel must reproduce, bit for
bit, what its two input kernels produce when launched one after the other (the reference's
check: tests/legacy main.cc compares run_fuse with run_kernel1/2 through check_matrix), and
those in turn are checked against numpy.
"""
import os

import numpy as np
import pytest

from bfuse_project_amd import config
from bfuse_project_amd._lib import BfuseError
from bfuse_project_amd.operation import GenericOperation, fill_uniform

pytestmark = pytest.mark.gpu

BUILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "frontend", "build")

# buffer shapes (I, F, O) of the test kernels
SHAPES = {
    "mm_tiled": [(128, 64), (64, 128), (128, 128)],
    "row_scale": [(128, 256), (128,), (128, 256)],
    "ew_max": [(10240,), (10240,), (10240,)],
}


def numpy_ref(name, I, F):
    if name == "mm_tiled":
        # the kernel adds products in k order in fp32; numpy's blocked sum differs in the last bits
        return (I.reshape(128, 64).astype(np.float64) @ F.reshape(64, 128).astype(np.float64)).ravel()
    if name == "row_scale":
        S = F.astype(np.float32)
        return (I.reshape(128, 256) * S[:, None] + np.roll(S, -1)[:, None]).astype(np.float32).ravel()
    return np.maximum(I, F)


def need(path):
    if not os.path.exists(path):
        pytest.fail(f"{path} missing: run `make -C tests/frontend` (or __graft_entry__.build()) before the GPU tests")
    return path


VARIANTS = [("zigzag", "bfuse"), ("ratio", "bfuse"), ("chunk8", "bfuse"), ("hfuse", "hfuse")]
PAIRS = [("mm_tiled", "row_scale"), ("mm_tiled", "ew_max")]


@pytest.mark.parametrize("k1,k2", PAIRS)
def test_emitted_kernels_match_unfused(k1, k2):
    _emitted_match_unfused((k1, k2), VARIANTS)


def test_emitted_kernels_of_three_match_unfused():
    _emitted_match_unfused(("mm_tiled", "row_scale", "ew_max"), [("zigzag3", "bfuse"), ("chunk8_3", "bfuse"), ("hfuse3", "hfuse")])


def _emitted_match_unfused(names, variants):
    kmap = config.load_kernels_yaml(os.path.join(os.path.dirname(BUILD), "kernels.yaml"))
    n = len(names)
    ins = []
    for side, k in enumerate(names):
        n_i, n_f = int(np.prod(SHAPES[k][0])), int(np.prod(SHAPES[k][1]))
        ins.append((fill_uniform(11 + side, n_i, -1.0, 1.0), fill_uniform(23 + side, n_f, -1.0, 1.0)))
    with GenericOperation(*[SHAPES[k] for k in names]) as op:
        for side in range(n):
            op.upload(side, *ins[side])
        unf = op.load(need(os.path.join(BUILD, "zigzag", "kernels.hsaco")))
        op.zero_outputs()
        for side, k in enumerate(names):
            op.launch(unf, k, kmap[k].GridDim, kmap[k].BlockDim, 3, side)
        base = [op.download(side) for side in range(n)]
        for side, k in enumerate(names):
            ref = numpy_ref(k, *ins[side])
            if k == "mm_tiled":
                np.testing.assert_allclose(base[side], ref, rtol=0, atol=1e-5 * np.sqrt(np.mean(ref ** 2)) * 8)
            else:
                assert np.array_equal(base[side], ref), k
        for folder, kind in variants:
            fused = config.load_kernels_yaml(need(os.path.join(BUILD, folder, f"{kind}_kernels.yaml")))
            name = "_".join(names) + f"_fused_{kind}"
            mod = op.load(need(os.path.join(BUILD, folder, "_".join(names) + f"_{kind}.hsaco")))
            op.zero_outputs()
            us = op.launch(mod, name, fused[name].GridDim, fused[name].BlockDim, 3 * n)
            assert us > 0
            for side in range(n):
                got = op.download(side)
                assert np.array_equal(got.view(np.uint32), base[side].view(np.uint32)), (folder, name, side)


def test_module_errors():
    with GenericOperation(SHAPES["mm_tiled"], SHAPES["ew_max"]) as op:
        with pytest.raises(BfuseError):
            op.load(os.path.join(BUILD, "no_such.hsaco"))
        mod = op.load(need(os.path.join(BUILD, "zigzag", "kernels.hsaco")))
        with pytest.raises(BfuseError, match="not in module"):
            op.launch(mod, "no_such_kernel", (1, 1, 1), (64, 1, 1), 3, 0)
        with pytest.raises(BfuseError):
            op.launch(mod, "ew_max", (1, 1, 1), (2048, 1, 1), 3, 1)
        with pytest.raises(BfuseError):
            op.launch(mod + 7, "ew_max", (1, 1, 1), (64, 1, 1), 3, 1)
