"""Weight layout: a bf16 weight held as [K, N] (the way the configuration writes pair 5's GEMM,
[512x4096].[4096x14336]) is brought into the GEMM's [N, K] operand layout by the library's transpose
kernel; checked byte for byte against numpy, at a small size and at the configuration's."""
import numpy as np
import pytest

import bfuse_project_amd as bf

pytestmark = pytest.mark.gpu


def _transpose_on_gpu(kernel, w_kn):
    with bf.Operation(kernel, "bias_relu_4096") as op:
        op.upload(0, w_kn, np.zeros(1, np.uint16))
        op.zero_outputs()
        op.launch("kernel1")
        out = op.download(0).copy()
        t = op.time("kernel1", warmup=5, reps=30)[0]
    return out, float(np.mean(t))


@pytest.mark.parametrize("kernel,rows,cols", [("transpose16_128x192", 128, 192), ("transpose16_4096x14336", 4096, 14336)])
def test_transpose_equals_numpy(kernel, rows, cols):
    print(kernel, flush=True)
    rng = np.random.default_rng(rows * 31 + cols)
    w = rng.integers(0, 65536, size=(rows, cols), dtype=np.uint16)
    got, us = _transpose_on_gpu(kernel, w)
    assert got.reshape(cols, rows).tobytes() == np.ascontiguousarray(w.T).tobytes()
    gbps = 2 * rows * cols * 2 / us * 1e-3
    print(f"{kernel}: {us:.1f} us, {gbps:.0f} GB/s", flush=True)


def test_pair5_gemm_from_a_weight_held_as_k_by_n():
    """The whole path a [K, N] weight takes: transpose on the device, then the GEMM; the result equals
    the GEMM over the weight generated in [N, K] directly."""
    from bfuse_project_amd.workloads import PAIRS
    print("pair 5 GEMM from a [K, N] weight", flush=True)
    pair = PAIRS[5]
    a, w_nk, x, f2 = pair.inputs()
    w_kn = np.ascontiguousarray(w_nk.reshape(14336, 4096).T)          # how the configuration writes it
    w_dev, _ = _transpose_on_gpu("transpose16_4096x14336", w_kn)
    assert w_dev.tobytes() == w_nk.tobytes()
    with bf.Operation(pair.k1, pair.k2) as op:
        want = op.run_kernel(0, a, w_nk)
        got = op.run_kernel(0, a, w_dev)
    assert got.tobytes() == want.tobytes()
