"""The give-up path of the per-side barrier (the gfx950 replacement for the reference's
`bar.sync id, n`, horizontal-fuser/src/Matchers.cc:288-320), forced from the host.

`selftest_sync_a` / `selftest_sync_b` are two-wave test operators whose wave 0 takes one barrier more
than wave 1 when they run under the side barrier.  The wait is bounded, so every kernel ends
normally; the host lowers the bound so that the give-up comes at once, and every entry point that
synchronises after such a launch must report BFUSE_ERR_SYNC -- once, with the counter cleared for
the next launch.
"""
import numpy as np
import pytest

import bfuse_project_amd as bf
from bfuse_project_amd._lib import BfuseError
from bfuse_project_amd.operation import fill_normal

pytestmark = pytest.mark.gpu

BFUSE_ERR_SYNC = -4


def _want(I, F):
    x = I.reshape(-1, 2, 64)[:, ::-1, :].reshape(-1)       # the two waves of a workgroup swap their values
    return x + F


def test_side_barrier_give_up_is_reported_by_every_synchronising_entry_point():
    I1, F1 = fill_normal(11, 512, 0, 1), fill_normal(12, 512, 0, 1)
    I2, F2 = fill_normal(13, 768, 0, 1), fill_normal(14, 768, 0, 1)
    with bf.Operation("selftest_sync_a", "selftest_sync_b") as op:
        # standalone (hardware barrier): well formed
        O1, O2 = op.run_kernel(0, I1, F1).ravel(), op.run_kernel(1, I2, F2).ravel()
        assert bool(np.array_equal(O1, _want(I1, F1))) and bool(np.array_equal(O2, _want(I2, F2)))
        fused = op.fused("hfuse")
        op.set_sync_spin_limit(fused, 64)
        try:
            print("[giveup] run_fuse", flush=True)
            with pytest.raises(BfuseError, match="side-barrier waits gave up") as ei:
                op.run_fuse(fused, I1, F1, I2, F2)
            assert ei.value.code == BFUSE_ERR_SYNC
            # asynchronous launch, then each call that synchronises
            op.upload(0, I1, F1)
            op.upload(1, I2, F2)
            print("[giveup] bfuse_launch + bfuse_synchronize", flush=True)
            op.zero_outputs()
            op.launch("hfuse", fused)
            with pytest.raises(BfuseError, match="gave up") as ei:
                op.synchronize()
            assert ei.value.code == BFUSE_ERR_SYNC
            op.synchronize()                                   # reported once; the counter was cleared
            # the matched barrier did its work: outputs are the unfused ones
            assert bool(np.array_equal(op.download(0).ravel(), O1)) and bool(np.array_equal(op.download(1).ravel(), O2))
            print("[giveup] bfuse_launch + bfuse_download", flush=True)
            op.launch("hfuse", fused)
            with pytest.raises(BfuseError, match="gave up"):
                op.download(0)
            print("[giveup] bfuse_time / bfuse_time_batched", flush=True)
            with pytest.raises(BfuseError, match="gave up"):
                op.time("hfuse", fused, warmup=1, reps=2)
            with pytest.raises(BfuseError, match="gave up"):
                op.time_batched("hfuse", fused, warmup=1, reps=2)
        finally:
            op.set_sync_spin_limit(fused, 1 << 22)
        op.synchronize()


def test_a_healthy_fused_kernel_after_a_give_up_is_clean():
    from tests.test_gpu_small import _cases
    cases = _cases()
    k1, k2 = "gemm_f32_128x160x192_d", "gemm_gelu_f32_64x192x288_d"      # both sides synchronise: side barriers on both
    I1, F1 = cases[k1][0](5)
    I2, F2 = cases[k2][0](6)
    with bf.Operation(k1, k2) as op:
        O1, O2 = op.run_kernel(0, I1, F1), op.run_kernel(1, I2, F2)
        Q1, Q2 = op.run_fuse(op.fused("hfuse"), I1, F1, I2, F2)             # raises on BFUSE_ERR_SYNC
        assert np.array_equal(Q1.view(np.uint8), O1.view(np.uint8)) and np.array_equal(Q2.view(np.uint8), O2.view(np.uint8))
