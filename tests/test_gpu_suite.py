"""Suite driver on the GPU: a 2 x 2 matrix of small kernels through every method, traces on
disk, speed-up table.  Validation inside the run is the reference's `-v` check tightened to
bit equality (main_cc.py:246-268)."""
import os

import pytest
import yaml

from bfuse_project_amd import suite

pytestmark = pytest.mark.gpu


def test_small_matrix(tmp_path):
    info_path = tmp_path / "info.yaml"
    info_path.write_text(yaml.safe_dump({"FusionSet": [{"Set": ["conv3x3_f32_32x12x12_32", "layernorm_8x256"]},
                                                       {"Set": ["gemm_gelu_f32_96x128x192", "softmax_causal_2x256x256"]}]}))
    info = suite.load_info(str(info_path))
    rows = suite.run_suite(info, str(tmp_path), validate=True, log=lambda m: print(m, flush=True))
    assert len(rows) == 4
    by = {(r["kernel1"], r["kernel2"]): r for r in rows}
    r = by[("conv3x3_f32_32x12x12_32", "gemm_gelu_f32_96x128x192")]
    assert r["bfuse_kernel"].startswith("conv3x3_f32_32x12x12_32_gemm_gelu_f32_96x128x192_fused_bfuse")
    assert r["serial_ns"] == pytest.approx(r["kernel1_ns"] + r["kernel2_ns"]) and r["bfuse_ns"] > 0 and r["parallel_ns"] > 0
    assert "bfuse_ns" in by[("layernorm_8x256", "softmax_causal_2x256x256")]
    assert "bfuse_ns" not in by[("layernorm_8x256", "gemm_gelu_f32_96x128x192")]      # no fused kernel built for it
    for stem in ("0_0_0", "1_0_1", "2_1_1", "4_0_0"):
        assert os.path.exists(tmp_path / "exec" / f"{stem}.csv")
    # the traces hold the warm-ups too; the analysis drops them
    assert len(suite.read_trace(str(tmp_path / "exec" / "0_0_0.csv"))) == suite.WARMUP_TRIALS + suite.TIMED_TRIALS
    print(suite.to_markdown(rows))


def test_from_a_user_config_to_the_speed_up_table(tmp_path):
    """The reference's front door end to end: operator ids and shapes in, resolved against the registry
    (configure), the pair matrix run and tabulated (suite)."""
    from bfuse_project_amd import configure
    cfg = tmp_path / "models.yaml"
    cfg.write_text("FusionSet:\n  - Set: [dense_3]\n  - Set: [conv2d_1, dense_0]\n"
                   "KernelInfo:\n  dense_3: [512, 768, 2304]\n  dense_0: [512, 512, 512]\n  conv2d_1: [1, 56, 56, 64, 64, 3, 3, 1, 1]\n")
    out = tmp_path / "suite"
    r = configure.configure(str(cfg), str(out))
    assert r["found"]["dense_3"] == "gemm_f32_512x768x2304"
    info = suite.load_info(str(out / "config" / "info.yaml"))
    print("suite from a user config", flush=True)
    rows = suite.run_suite(info, str(out / "run"), validate=True, log=lambda m: print(m, flush=True))
    assert [(x["kernel1"], x["kernel2"]) for x in rows] == [("gemm_f32_512x768x2304", "conv3x3_f32_64x56x56_64"),
                                                             ("gemm_f32_512x768x2304", "gemm_f32_512x512x512")]
    assert all(x["serial_ns"] > 0 and x["parallel_ns"] > 0 for x in rows)


def test_quick_start_command(tmp_path):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = tmp_path / "m.yaml"
    cfg.write_text("FusionSet:\n  - Set: [dense_3]\n  - Set: [conv2d_1]\nKernelInfo:\n  dense_3: [512, 768, 2304]\n  conv2d_1: [1, 56, 56, 64, 64, 3, 3, 1, 1]\n")
    out = tmp_path / "qs"
    print("quick_start", flush=True)
    r = subprocess.run([sys.executable, "-m", "bfuse_project_amd.quick_start", str(cfg), "-o", str(out)], capture_output=True, text=True, cwd=root, timeout=120)
    assert r.returncode == 0, r.stdout[-1500:] + r.stderr[-1500:]
    assert "[1/3]" in r.stdout and "[3/3]" in r.stdout and "gemm_f32_512x768x2304" in r.stdout
    assert os.path.exists(out / "summary.md") and os.path.exists(out / "config" / "kernels.yaml") and os.path.exists(out / "exec" / "2_0_0.csv")
    with open(out / "exec_figure.png", "rb") as f:      # the reference's [6/6]: its speed-up figure
        assert f.read(4) == b"\x89PNG"
    # a second run into the same directory is refused, as the reference's configure step refuses it
    r = subprocess.run([sys.executable, "-m", "bfuse_project_amd.quick_start", str(cfg), "-o", str(out)], capture_output=True, text=True, cwd=root, timeout=120)
    assert r.returncode == 1 and "already exists" in r.stderr
