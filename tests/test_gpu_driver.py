"""The C++ command-line driver (the reference's `benchmark [-v] [-n N] T K1 K2`) end to end on
the GPU: every mode validates, and a mismatch would exit with status 1 as the reference's does."""
import os
import subprocess

import pytest

from tests.perf_report import expect

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "bfuse-project_amd", "benchmark")


def _run(*args):
    print("benchmark", *args, flush=True)
    return subprocess.run([EXE, *args], capture_output=True, text=True, timeout=120)


def test_driver_modes_validate():
    if not os.path.exists(EXE):
        pytest.fail(f"{EXE} has not been built")
    k1, k2 = "gemm_f32_512x768x2304", "layernorm_512x768"
    for mode, extra in (("0", []), ("1", []), ("2", []), ("5", []), ("4", ["-x", "_r"])):
        r = _run("-v", "-n", "5", *extra, mode, k1, k2)
        assert r.returncode == 0, r.stdout + r.stderr
        assert "INVALID" not in r.stdout and "VALID" in r.stdout
    r = _run("-v", "-n", "3", "3", "gemm_f32_512x512x512", "bias_relu_1048576")
    assert r.returncode == 0 and "bit-exact: yes" in r.stdout, r.stdout + r.stderr
    # bf16 pair with the packed byte operand
    r = _run("-v", "-n", "2", "-x", "_c256", "4", "gemm_bf16_512x4096x14336", "rmsnorm_rope_bf16_512x4096")
    assert r.returncode == 0 and "bit-exact: yes" in r.stdout, r.stdout + r.stderr


def test_driver_takes_positions_in_the_suites_info_yaml(tmp_path):
    """Three commands of the reference's matrix (`benchmark -v T idx1 idx2`, scripts/profile_test_suite.py:13-47)
    over a `configure` output: the positions select the members of info.yaml's two sets."""
    import yaml
    from bfuse_project_amd import configure
    out = tmp_path / "s"
    configure.configure(os.path.join(ROOT, "bfuse-project_amd", "examples", "model_operators.yaml"), str(out))
    info_path = str(out / "config" / "info.yaml")
    with open(info_path) as f:
        sets = [s["Set"] for s in yaml.safe_load(f)["FusionSet"]]
    for t, i, j in ((0, 3, 0), (2, 1, 2), (4, 3, 4)):
        r = _run("-v", "-n", "3", "-i", info_path, str(t), str(i), str(j))
        assert r.returncode == 0, r.stdout + r.stderr
        assert f"- Kernel1: {sets[0][i]}\n" in r.stdout and f"- Kernel2: {sets[1][j]}\n" in r.stdout
        assert "INVALID" not in r.stdout and "VALID" in r.stdout
        if t == 4:
            assert f"- Fused kernel: {sets[0][i]}_{sets[1][j]}_fused_bfuse" in r.stdout and "bit-exact: yes" in r.stdout
    r = _run("-v", "4", "3", "4")          # the same positions without the info file
    assert r.returncode != 0 and "info.yaml" in r.stderr


def test_driver_rejects_unknown_kernels():
    r = _run("4", "no_such_kernel", "layernorm_512x768")
    assert r.returncode != 0 and "unknown kernel" in r.stderr


def test_placement_probe_shows_the_round_robin_the_dispatch_patterns_rely_on():
    """Consecutive workgroup ids go to consecutive XCDs (starting wherever the hardware's round-robin
    stands), and an XCD deals its share evenly over
    its CUs -- why chunk = 256 (one chunk per round over all CUs) is the pattern used here and
    why the 1:1 zig-zag parks one operator on the even XCDs."""
    import numpy as np
    from bfuse_project_amd.operation import probe_placement
    p = probe_placement(512, 256, 3000)
    # round-robin over the eight XCDs; the XCD the first workgroup lands on depends on where the
    # previous dispatch stopped, so only the rotation is fixed
    assert np.all((p["xcc"].astype(np.int64) - int(p["xcc"][0])) % 8 == np.arange(512) % 8)
    key = p["xcc"].astype(np.int64) * 10000 + p["se"].astype(np.int64) * 100 + p["cu"]
    cus, counts = np.unique(key, return_counts=True)
    assert len(cus) <= 256
    expect(len(cus) == 256 and counts.min() == 2 and counts.max() == 2,
           f"512 workgroups on {len(cus)} CUs, {counts.min()} to {counts.max()} per CU (two each on an idle chip)")
    with pytest.raises(Exception):
        probe_placement(0)


@pytest.mark.parametrize("name,flops,nominal", [("mfma_stream_bf16_2000", 256 * 8 * 14 * 2000 * 16384.0, 2500.0),
                                                 ("mfma_stream_f32_1000", 256 * 8 * 14 * 1000 * 2048.0, 157.3)])
def test_mfma_only_kernels_give_a_ceiling_below_the_published_peak(name, flops, nominal):
    """The measured-ceiling kernels of the bench line: the same bytes on every launch, finite and not all
    zero, and a rate between a third of the published peak and the peak itself."""
    import numpy as np
    import bfuse_project_amd as bf
    print(name, flush=True)
    with bf.Operation(name, "bias_relu_4096") as op:
        z = np.zeros(1, np.float32)
        op.upload(0, z, z)
        op.zero_outputs()
        op.launch("kernel1")
        a = op.download(0).copy()
        op.zero_outputs()
        op.launch("kernel1")
        b = op.download(0)
        t = op.time("kernel1", warmup=5, reps=20)[0]
    assert a.size == 256 * 512 and np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.all(np.isfinite(a)) and np.count_nonzero(a) > a.size // 2
    tflops = flops / float(np.mean(t)) * 1e-6
    print(f"{name}: {tflops:.1f} TFLOP/s of {nominal}", flush=True)
    assert tflops > 0
    expect(nominal / 3 < tflops <= nominal * 1.02, f"{name}: {tflops:.1f} TFLOP/s of the published {nominal}")


def test_shutdown_releases_everything_and_the_library_can_be_initialized_again():
    """bfuse_shutdown with a side still live and a launch still queued: it waits, frees the buffers, and a
    later bfuse_init + operation works as before."""
    import numpy as np
    import bfuse_project_amd as bf
    from bfuse_project_amd import _lib
    print("shutdown / re-init", flush=True)
    x = np.arange(4096, dtype=np.float32) - 2048.0
    b = np.ones(4096, np.float32)
    op = bf.Operation("bias_relu_4096", "layernorm_8x256")
    op.upload(0, x, b)
    op.launch("kernel1")
    _lib.check(_lib.lib().bfuse_shutdown())          # side buffers of `op` are gone now
    op.live = False
    _lib.check(_lib.lib().bfuse_shutdown())          # twice is harmless
    with bf.Operation("bias_relu_4096", "layernorm_8x256") as op2:
        op2.upload(0, x, b)
        op2.zero_outputs()
        op2.launch("kernel1")
        y = op2.download(0)
    assert np.array_equal(y.ravel(), np.maximum(x + b, 0.0))


def test_clock_stamped_gemm_computes_what_the_product_kernel_computes():
    """The instrumented instance of pair 5's GEMM (clock stamps behind its output matrix) is the product kernel
    plus counter reads: the matrix must be byte-identical, alone and with the norm waves fused in, and the stamps
    ordered (loop start < loop end < last store acknowledged) on eight XCDs; the table of
    `python -m bfuse_project_amd.profile_pair --clock` comes out of them."""
    import numpy as np
    import bfuse_project_amd as bf
    from bfuse_project_amd.profile_pair import clock_table
    from bfuse_project_amd.workloads import PAIRS
    print("clock-stamped GEMM", flush=True)
    I1, F1, I2, F2 = PAIRS[5].inputs()
    with bf.Operation("gemm_bf16_512x4096x14336", "rmsnorm_rope_bf16_512x4096_w2") as op:
        want = op.run_kernel(0, I1, F1)
        want2 = op.run_kernel(1, I2, F2)
    with bf.Operation("gemm_bf16_512x4096x14336_clk", "rmsnorm_rope_bf16_512x4096_w2") as op:
        got = op.run_kernel(0, I1, F1)
        q1, q2 = op.run_fuse(op.fused("hfuse"), I1, F1, I2, F2)
    n = 512 * 14336
    assert np.array_equal(got.ravel()[:n], want.ravel()) and np.array_equal(q1.ravel()[:n], want.ravel()) and np.array_equal(q2, want2)
    st = got.ravel().view(np.uint8)[n * 2:].view(np.uint64).reshape(256, 8).astype(np.int64)
    assert np.all(st[:, 0] < st[:, 1]) and np.all(st[:, 1] < st[:, 2]) and np.all(st[:, 3] <= st[:, 4]) and np.all(st[:, 4] <= st[:, 5])
    assert sorted(set((st[:, 6] & 15).tolist())) == list(range(8))
    table = clock_table(20)
    print(table, flush=True)
    assert "shader clocks per K-stage" in table and table.count("| 7 |") == 2


def test_scheduler_probe_reports_the_mix_of_two_operators_per_cu_and_xcd():
    """The reference's scheduler experiment (tests/interleave_scheduler/test/test_scheduler.py) on this chip: under
    the 1:1 interleave every XCD, and so every CU, sees one operator only; in chunks of 256 every XCD sees both
    alike.  (What an XCD receives follows from id % 8 and is asserted; how an XCD spreads its workgroups over its
    CUs while others are resident is the hardware's business and is printed.)"""
    import numpy as np
    from bfuse_project_amd import scheduler_probe as sp
    print("scheduler probe: zigzag", flush=True)
    z = sp.probe("zigzag", (2048, 2048), 256, 1, 1)
    assert z["fused_grid"] == 4096 and z["side"].size == 4096 and z["cu"].max() <= 255
    zx = sp.mix_statistics(z["xcd"], z["side"])
    assert zx["units"] == 8 and zx["mean_diff"] == 1.0
    assert sp.mix_statistics(z["cu"], z["side"])["mean_diff"] == 1.0
    print(sp.report(z, color=False), flush=True)
    print("scheduler probe: chunked", flush=True)
    c = sp.probe("chunked", (2048, 2048), 256, 256, 1)
    cx = sp.mix_statistics(c["xcd"], c["side"])
    assert cx["mean_diff"] == 0.0 and np.all(cx["n0"] == 256) and np.all(cx["n1"] == 256)
    cc = sp.mix_statistics(c["cu"], c["side"])
    print(sp.report(c, color=False), flush=True)
    assert cc["mean_diff"] < 0.5
    assert sp.main(["--pattern", "ranges", "--grids", "512", "256", "--first", "600", "--rows", "3", "--no-color"]) == 0
