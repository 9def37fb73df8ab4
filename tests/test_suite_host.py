"""Suite driver, host side: the command matrix and the trace statistics.

The statistics restate scripts/analyze_test_suite.py:103-161 and are checked on traces whose
answers are known by construction, and on rows in the reference's own nsys export format.
"""
import os

import numpy as np
import pytest
import yaml

import bfuse_project_amd as bf

from bfuse_project_amd import suite

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture
def info(tmp_path):
    p = tmp_path / "info.yaml"
    p.write_text(yaml.safe_dump({"FusionSet": [{"Set": ["a0", "a1", "a2"]}, {"Set": ["b0", "b1", "b2", "b3"]}],
                                 "KernelInfo": {"a0": [1, 2, 3]}}))
    return suite.load_info(str(p))


def test_info_must_have_two_sets(tmp_path):
    p = tmp_path / "bad.yaml"
    p.write_text(yaml.safe_dump({"FusionSet": [{"Set": ["a"]}]}))
    with pytest.raises(ValueError, match="only 2"):
        suite.load_info(str(p))
    assert suite.main([str(p)]) == 1
    p.write_text(yaml.safe_dump({"FusionSet": [{"Set": ["a"]}, {"Set": []}]}))
    with pytest.raises(ValueError):
        suite.load_info(str(p))


def test_command_matrix_follows_the_reference(info):
    # kernel1: one per first-set member; kernel2: one per second-set member; the three two-kernel
    # methods: one per pair (profile_test_suite.py:33-45), upper triangle on request
    full = suite.exec_commands(info, "/x/benchmark", "/out/exec")
    assert len(full) == 3 + 4 + 3 * 12
    tri = suite.exec_commands(info, "/x/benchmark", "/out/exec", triangular=True)
    assert len(tri) == 3 + 4 + 3 * (4 + 3 + 2)
    c = full[0]
    assert c[:2] == ["rocprofv3", "--kernel-trace"] and c[c.index("--") + 1:] == ["/x/benchmark", "-n", "33", "0", "a0", "b0"]
    assert full[3 + 4][-3:] == ["2", "a0", "b0"] and "-o" in c and c[c.index("-o") + 1] == "0_0_0"
    last = full[-1]
    assert last[-3:] == ["4", "a2", "b3"] and last[last.index("-o") + 1] == "4_2_3"
    v = suite.valid_commands(info, "/x/benchmark")
    assert all(x[1] == "-v" for x in v) and len(v) == len(full)
    # operators of several GB: the driver's resident mode in every command
    r = suite.exec_commands(info, "/x/benchmark", "/out/exec", resident=True)
    assert r[0][r[0].index("--") + 1:] == ["/x/benchmark", "-n", "33", "-r", "0", "a0", "b0"]
    assert all(x[1:3] == ["-v", "-r"] for x in suite.valid_commands(info, "/x/benchmark", resident=True))


def test_single_and_parallel_statistics():
    rows = []
    t = 0.0
    for r in range(33):
        rows.append({"Name": "k", "Start": t, "Duration": 100.0 + r})       # 100..132
        rows.append({"Name": "other", "Start": t + 1, "Duration": 5.0})
        t += 1000
    mn, mx, mean, std = suite.single_statistics(rows, "k")
    assert (mn, mx) == (103.0, 132.0) and mean == pytest.approx(np.mean(np.arange(103, 133))) and std == pytest.approx(np.std(np.arange(103, 133)))
    with pytest.raises(ValueError):
        suite.single_statistics(rows, "missing")
    # two kernels per repetition: second ends later -> span; first ends later -> its duration
    rows, t = [], 0.0
    for r in range(5):
        rows.append({"Name": "a", "Start": t, "Duration": 50.0})
        rows.append({"Name": "b", "Start": t + 10, "Duration": 60.0 if r != 4 else 20.0})
        t += 500
    mn, mx, mean, std = suite.parallel_statistics(rows, ["a", "b"], warmup=3)
    assert (mn, mx) == (50.0, 70.0) and mean == 60.0
    with pytest.raises(ValueError, match="must be 2"):
        suite.parallel_statistics(rows, ["a"])


def test_trace_formats(tmp_path):
    own = tmp_path / "0_0_0.csv"
    suite.write_trace(str(own), [{"Name": "k", "Start": 5.0, "Duration": 7.0}, {"Name": "k", "Start": 1.0, "Duration": 3.0}])
    assert [r["Start"] for r in suite.read_trace(str(own))] == [1.0, 5.0]
    roc = tmp_path / "roc_kernel_trace.csv"
    roc.write_text('"Kind","Agent_Id","Queue_Id","Kernel_Name","Start_Timestamp","End_Timestamp"\n'
                   '"KERNEL_DISPATCH",1,1,"k",1000,1800\n"KERNEL_DISPATCH",1,1,"k",3000,3900\n')
    assert [(r["Name"], r["Duration"]) for r in suite.read_trace(str(roc))] == [("k", 800.0), ("k", 900.0)]
    # the reference's nsys export: memcpy rows have a duration too, kernels are picked by name later
    nsys = tmp_path / "nsys.csv"
    nsys.write_text("Start (ns),Duration (ns),CorrId,GrdX,Name\n288325122,257825,241,,[CUDA memcpy Host-to-Device]\n"
                    "289000000,41000,250,768,dense1_0_dense2_0_fused_bfuse\n")
    rows = suite.read_trace(str(nsys))
    assert rows[-1] == {"Name": "dense1_0_dense2_0_fused_bfuse", "Start": 289000000.0, "Duration": 41000.0}


def test_analyze_and_tables(tmp_path, info):
    exec_dir = tmp_path / "exec"
    exec_dir.mkdir()

    def trace(name, dur, n=33):
        return [{"Name": name, "Start": 1000.0 * r, "Duration": dur} for r in range(n)]
    suite.write_trace(str(exec_dir / "0_0_0.csv"), trace("a0", 100.0))
    suite.write_trace(str(exec_dir / "1_0_1.csv"), trace("b1", 50.0))
    suite.write_trace(str(exec_dir / "4_0_1.csv"), trace("a0_b1_fused_bfuse_c256", 120.0))
    suite.write_trace(str(exec_dir / "3_0_1.csv"), trace("a0_b1_fused_hfuse", 125.0))
    par = []
    for r in range(33):
        par += [{"Name": "a0", "Start": 1000.0 * r, "Duration": 100.0}, {"Name": "b1", "Start": 1000.0 * r + 5, "Duration": 50.0}]
    suite.write_trace(str(exec_dir / "2_0_1.csv"), par)
    rows = suite.analyze(info, str(exec_dir))
    assert len(rows) == 1
    r = rows[0]
    assert r["serial_ns"] == 150.0 and r["bfuse_speedup"] == pytest.approx(1.25) and r["hfuse_speedup"] == pytest.approx(1.2)
    assert r["parallel_ns"] == 100.0 and r["bfuse_kernel"] == "a0_b1_fused_bfuse_c256"
    md = suite.to_markdown(rows)
    assert "geomean speed-up over serial" in md and "1.25x" in md
    assert suite.geomean([2.0, 8.0]) == pytest.approx(4.0)
    assert suite.main([os.path.join(ROOT, "bfuse-project_amd", "examples", "headline_pairs.yaml"), "--commands", "-o", str(tmp_path)]) == 0


# ---- numeric K1 / K2 of the command-line driver ----------------------------------------------
EXE = os.path.join(ROOT, "bfuse-project_amd", "benchmark")


def _dry(args, cwd=None):
    import subprocess
    r = subprocess.run([EXE, "-d", *args], capture_output=True, text=True, timeout=60, cwd=cwd)
    got = {}
    for line in r.stdout.splitlines():
        if line.startswith("- ") and ": " in line:
            k, v = line[2:].split(": ", 1)
            got[k] = v.split()[0] if k == "Fused kernel" else v
    return r, got


def test_numeric_ids_are_positions_in_the_suites_info_yaml(tmp_path):
    """The reference's command matrix (scripts/profile_test_suite.py:13-47) passes positions in the two
    FusionSets of info.yaml, and its benchmark switches on them (macro_h.py:296-320).  Restated here for
    a `configure` output and resolved command by command (dry run: needs no device)."""
    from bfuse_project_amd import configure, tuner
    out = tmp_path / "s"
    configure.configure(os.path.join(ROOT, "bfuse-project_amd", "examples", "model_operators.yaml"), str(out))
    info_path = str(out / "config" / "info.yaml")
    with open(info_path) as f:
        info_yaml = yaml.safe_load(f)
    fusion_sets = info_yaml["FusionSet"]
    kernel1_size, kernel2_size = len(fusion_sets[0]["Set"]), len(fusion_sets[1]["Set"])
    assert kernel1_size >= 2 and kernel2_size >= 2 and fusion_sets[0]["Set"] != fusion_sets[1]["Set"]
    # the reference's loops, upper triangle included
    want = []
    for idx in range(5):
        if idx == 0:
            want += [[str(idx), str(k), "0"] for k in range(kernel1_size)]
        if idx == 1:
            want += [[str(idx), "0", str(k)] for k in range(kernel2_size)]
        if idx in (2, 3, 4):
            want += [[str(idx), str(k1), str(k2)] for k1 in range(kernel1_size) for k2 in range(k1, kernel2_size)]
    ours = suite.valid_commands(suite.load_info(info_path), EXE, triangular=True, info_path=info_path)
    assert [c[-3:] for c in ours] == want
    assert all(c[:4] == [EXE, "-v", "-i", info_path] for c in ours)
    checked_fused = 0
    for c in ours:
        t, i, j = int(c[-3]), int(c[-2]), int(c[-1])
        k1, k2 = fusion_sets[0]["Set"][i], fusion_sets[1]["Set"][j]
        built = tuner.built_variants(k1, k2)
        if t in (3, 4) and not [h for h in built if h.kind == (2 if t == 3 else 1)]:
            r, got = _dry(c[2:])
            assert r.returncode != 0 and "unknown kernel" in r.stderr      # no fused kernel of that kind for the pair
            continue
        r, got = _dry(c[2:])
        assert r.returncode == 0, (c, r.stderr)
        assert got["Kernel1"] == k1 and got["Kernel2"] == k2, (c, got)
        if t in (3, 4):
            h = bf.kernel_info(got["Fused kernel"])
            assert h.sides == (k1, k2) and h.kind == (2 if t == 3 else 1)
            checked_fused += 1
    assert checked_fused >= 4


def test_numeric_ids_without_an_info_file_are_an_error_and_names_keep_working(tmp_path):
    r, _ = _dry(["4", "0", "1"], cwd=str(tmp_path))
    assert r.returncode != 0 and "info.yaml" in r.stderr
    r, got = _dry(["4", "gemm_f32_512x768x2304", "layernorm_512x768"], cwd=str(tmp_path))
    assert r.returncode == 0 and got["Fused kernel"] == "gemm_f32_512x768x2304_layernorm_512x768_fused_bfuse"
    # ./config/info.yaml is the default; flow-style lists and quoted names are read too
    (tmp_path / "config").mkdir()
    (tmp_path / "config" / "info.yaml").write_text(
        "# suite\nFusionSet:\n  - Set: [bias_relu_4096, 'gemm_f32_512x768x2304']\n  - Set:\n      - layernorm_8x256\n      - layernorm_512x768\n"
        "KernelInfo:\n  dense_3: [512, 768, 2304]\n")
    r, got = _dry(["4", "1", "1"], cwd=str(tmp_path))
    assert r.returncode == 0 and (got["Kernel1"], got["Kernel2"]) == ("gemm_f32_512x768x2304", "layernorm_512x768")
    r, got = _dry(["0", "0", "0"], cwd=str(tmp_path))
    assert r.returncode == 0 and (got["Kernel1"], got["Kernel2"]) == ("bias_relu_4096", "layernorm_8x256")
    r, _ = _dry(["0", "2", "0"], cwd=str(tmp_path))
    assert r.returncode != 0 and "out of range" in r.stderr
    one = tmp_path / "one.yaml"
    one.write_text("FusionSet:\n- Set:\n  - bias_relu_4096\n")
    r, _ = _dry(["-i", str(one), "0", "0", "0"], cwd=str(tmp_path))
    assert r.returncode != 0 and "only 2" in r.stderr


def test_speedup_statistics_and_figure(tmp_path):
    """The block the reference prints under its speed-up figure (scripts/analyze_test_suite.py:1203-1209: max, min,
    geometric mean, standard deviation per form) and the figure itself, over rows written down here."""
    import json
    rows = [{"kernel1": "a", "kernel2": "b", "parallel_speedup": 1.0, "hfuse_speedup": 0.5, "bfuse_speedup": 2.0, "chooser_speedup": 2.0},
            {"kernel1": "a", "kernel2": "c", "parallel_speedup": 1.21, "bfuse_speedup": 0.5, "chooser_speedup": 1.0}]
    rows += [{"kernel1": "x", "kernel2": str(i), "parallel_speedup": 1.0, "bfuse_speedup": 1.0, "chooser_speedup": 1.0} for i in range(25)]
    st = suite.speedup_statistics(rows)
    assert st["hfuse"] == {"pairs": 1, "max": 0.5, "min": 0.5, "avg": 0.5, "std": 0.0}
    assert st["bfuse"]["pairs"] == 27 and st["bfuse"]["max"] == 2.0 and st["bfuse"]["min"] == 0.5
    assert st["bfuse"]["avg"] == pytest.approx(1.0)                      # 2 x 0.5 x 1 ... = 1
    assert st["parallel"]["avg"] == pytest.approx(1.21 ** (1 / 27))
    assert st["chooser"]["avg"] == pytest.approx(2.0 ** (1 / 27)) and "serial" not in st
    path = suite.draw_speedup_figure(rows, str(tmp_path / "exec_figure.png"))      # 27 pairs: two rows of the figure
    with open(path, "rb") as f:
        assert f.read(8) == b"\x89PNG\r\n\x1a\n"
    assert suite.speedup_statistics([]) == {}
