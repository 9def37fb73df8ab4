"""Host logic that needs no GPU: the YAML wire format, FusionContext naming/shape, and that the
C-ABI library loads and exports every symbol include/bfuse_rt.h declares."""
import ctypes
import os
import re

import pytest
import yaml

import bfuse_project_amd as bf
from bfuse_project_amd import _lib, config

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_declared_symbol_is_exported():
    header = open(os.path.join(ROOT, "include", "bfuse_rt.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", header)) - {"defined", "sizeof", "void"}
    declared = {d for d in declared if not d.isupper() and not d.endswith("_fn")}
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"libbfuse_rt.so does not export {name}"


def test_the_header_is_plain_c_and_the_group_example_compiles(tmp_path):
    """include/bfuse_rt.h must be usable from C (the reference's harness is C-callable) and the
    three-kernel binding shown to maintainers must compile against it."""
    import shutil
    import subprocess
    if not shutil.which("gcc"):
        pytest.skip("no gcc")
    hdr = os.path.join(ROOT, "include", "bfuse_rt.h")
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c", hdr])
    src = tmp_path / "group.c"
    src.write_text('''
#include <stdio.h>
#include "bfuse_rt.h"
int run(const void* I[3], const void* F[3], void* O[3]) {
    bfuse_kernel_info k[3], fused;
    const char* names[3] = {"gemm_f32_512x768x2304_s2", "layernorm_512x768", "softmax_causal_12x512x512"};
    int i;
    for (i = 0; i < 3; ++i) {
        if (bfuse_kernel_find(names[i], &k[i])) return 1;
        bfuse_set_elem_bytes(i + 1, k[i].elem_bytes[0], k[i].elem_bytes[1], k[i].elem_bytes[2]);
        if (bfuse_initialize_side(i + 1, k[i].shape[0], k[i].shape[1], k[i].shape[2])) return 2;
        bfuse_upload(i + 1, I[i], F[i]);
    }
    if (bfuse_kernel_find("gemm_f32_512x768x2304_s2_layernorm_512x768_softmax_causal_12x512x512_fused_bfuse_c256", &fused)) return 3;
    {
        bfuse_launch_desc d = {fused.func, {fused.grid[0], 1, 1}, {fused.block[0], 1, 1}, fused.n_sides, {1, 2, 3, 0}};
        float us_each, us_queued;
        if (bfuse_launch_list(1, &d) || bfuse_time_list(1, &d, 20, 300, &us_each, &us_queued)) { fprintf(stderr, "%s\\n", bfuse_last_error()); return 4; }
    }
    for (i = 0; i < 3; ++i) { bfuse_download(i + 1, O[i]); bfuse_finalize_side(i + 1); }
    return 0;
}
''')
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src), "-o", str(tmp_path / "group.o")])


def test_registry_lists_pairs_and_fused_names_follow_the_reference():
    ks = {k.name: k for k in bf.list_kernels()}
    from bfuse_project_amd.workloads import PAIRS, fusions
    for pair in PAIRS.values():
        for (k1, k2), variants in fusions(pair).items():
            assert ks[k1].kind == 0 and ks[k2].kind == 0
            for kind, suffix in variants:
                f = ks[f"{k1}_{k2}_fused_{kind}{suffix}"]          # Contexts.cc:56-92 naming
                assert f.sides == (k1, k2)
                d = [bf.LaunchDims(ks[k1].grid, ks[k1].block), bf.LaunchDims(ks[k2].grid, ks[k2].block)]
                if kind == "bfuse":
                    names = {0: "zigzag", 1: "proportional", 2: "chunked", 3: "ranges"}
                    plan = bf.plan_blocks(names[f.pattern], d, max(f.p0, 1), max(f.p1, 1))
                else:
                    plan = bf.plan_threads(d, pad=64)
                assert (f.grid[0], f.block[0]) == (plan.fused_grid, plan.fused_block), f.name
                assert f.block[0] % 64 == 0


def test_device_entry_points_fail_loudly_without_a_gpu():
    import subprocess
    import sys
    code = ("import ctypes, sys; sys.path.insert(0, %r); from bfuse_project_amd import _lib; l = _lib.lib();"
            "rc = l.bfuse_init(0); print(rc, l.bfuse_last_error().decode())" % ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env={**os.environ, "HIP_VISIBLE_DEVICES": "-1"})
    rc = int(out.stdout.split()[0])
    if rc == 0:
        pytest.skip("a GPU is visible to this process")
    assert rc == -2 and "no CPU path" in out.stdout


def test_launch_lists_and_generic_sides_refuse_work_before_init():
    """No compute call without a device: the entry points for more than two kernels return an error
    state (not a crash) when bfuse_init has not succeeded."""
    import subprocess
    import sys
    code = ("import ctypes as C, sys; sys.path.insert(0, %r); from bfuse_project_amd import _lib; l = _lib.lib();"
            "d = (_lib.LaunchDescC * 1)(); s = (C.c_int * 4)(1, 1, 1, 1); us = C.c_float();"
            "print(l.bfuse_launch_list(1, d), l.bfuse_time_list(1, d, 1, 1, C.byref(us), C.byref(us)),"
            " l.bfuse_initialize_side(3, s, s, s), l.bfuse_initialize_side(5, s, s, s), l.bfuse_finalize_side(0))" % ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env={**os.environ, "HIP_VISIBLE_DEVICES": "-1"})
    rcs = [int(x) for x in out.stdout.split()]
    assert len(rcs) == 5 and all(rc < 0 for rc in rcs), (out.stdout, out.stderr[-500:])


def test_null_plans_and_shutdown_before_init_are_errors_not_crashes():
    import ctypes as C
    from bfuse_project_amd import _lib
    l = _lib.lib()
    v = C.c_int(7)
    assert l.bfuse_map_block(None, 0, C.byref(v)) == -1 and v.value == -1
    v = C.c_int(7)
    assert l.bfuse_map_thread(None, 0, 0, C.byref(v)) == -1 and v.value == -1
    assert b"null plan" in l.bfuse_last_error()
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); from bfuse_project_amd import _lib; l = _lib.lib(); print(l.bfuse_shutdown(), l.bfuse_shutdown())" % ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env={**os.environ, "HIP_VISIBLE_DEVICES": "-1"})
    assert out.stdout.split() == ["0", "0"], (out.stdout, out.stderr[-500:])


def test_reference_yaml_files_load(golden_dir):
    d = os.path.join(golden_dir, "config_sample")
    kernels = bf.load_kernels_yaml(os.path.join(d, "kernels.yaml"))          # written by PyYAML
    fusions = bf.load_fusions_yaml(os.path.join(d, "fusions.yaml"))
    bfk = bf.load_kernels_yaml(os.path.join(d, "bfuse_kernels.yaml"))        # written by llvm::yaml
    hfk = bf.load_kernels_yaml(os.path.join(d, "hfuse_kernels.yaml"))
    assert kernels["conv2d_4"].BlockDim == (19, 1, 8) and kernels["conv2d_4"].ExecTime == -1
    assert fusions[0].Kernels == ["bgemm_0", "conv2d_4"] and fusions[0].File == "kernels.cu"
    # the reference built this case with M = 2, N = 1 and 32-thread padding
    b = bf.FusionContext.create(fusions[0], kernels, bfuse=True, pattern="zigzag", p0=2, p1=1)
    h = bf.FusionContext.create(fusions[0], kernels, bfuse=False, pad=32)
    for ctx, ref in ((b, bfk), (h, hfk)):
        got = ctx.fused_kernel_info()
        want = ref[ctx.FusedKernelName]
        assert (got.KernelName, got.GridDim, got.BlockDim, got.Reg, got.HasBarriers) == \
               (want.KernelName, want.GridDim, want.BlockDim, want.Reg, want.HasBarriers)
    # on gfx950 the same pair pads the 152-thread side to whole wavefronts: 64 + 192
    h64 = bf.FusionContext.create(fusions[0], kernels, bfuse=False)
    assert h64.FusedBlockDim == (256, 1, 1) and h64.plan.thr_lo == [0, 64]


def test_yaml_roundtrip_and_errors(tmp_path):
    infos = {"a": bf.KernelInfo("a", True, (2, 3, 4), (8, 16, 1), 32), "b": bf.KernelInfo("b", False, (7, 1, 1), (64, 1, 1), 100, 12.5)}
    p = tmp_path / "k.yaml"
    bf.dump_kernels_yaml(infos, p)
    again = bf.load_kernels_yaml(p)
    assert again == infos
    assert "ExecTime" not in yaml.safe_load(open(p))["a"]             # optional key, default -1 (Utils.h:80)
    with pytest.raises(ValueError):
        config.parse_kernels({"a": {"KernelName": "a", "GridDim": {"X": 1, "Y": 1, "Z": 1}}})   # missing required keys
    with pytest.raises(ValueError):
        config.parse_kernels(["not", "a", "map"])
    with pytest.raises(ValueError):
        config.parse_fusions({"File": "x"})
    with pytest.raises(KeyError):                                      # unknown kernel, like map::at (Contexts.cc:69)
        bf.FusionContext.create(bf.FusionInfo("k.cu", ["a", "zzz"]), infos, bfuse=True)


def test_choose_fusion_uses_footprints():
    gemm = bf.KernelInfo("gemm", True, (256, 1, 1), (256, 1, 1), 232)
    ln = bf.KernelInfo("ln", False, (512, 1, 1), (64, 1, 1), 48)
    c = config.choose_fusion(gemm, ln, lds_a=73728, lds_b=0)
    assert c["hfuse_ok"] and c["prefer"] == "bfuse" and c["wg_per_cu"][0] == 2
    both = config.choose_fusion(gemm, gemm, 73728, 98304)
    assert not both["hfuse_ok"]                                        # two barrier-bearing sides -> block fusion
    big = config.choose_fusion(bf.KernelInfo("g", True, (256, 1, 1), (256, 1, 1), 300), ln, 98304, 0)
    assert big["wg_per_cu"][0] == 1                                    # > 256 VGPRs: nothing fits next to it


def test_traffic_figures_come_out_of_the_profile_summaries_of_the_registered_kernels():
    """`roofline.traffic` of the benchmark line is read from the traffic table of the fused kernel's profile
    summary: every headline kernel is registered, has a summary, and the summary has a row for it with a figure
    between the pair's algorithmic bytes and three times that."""
    from bfuse_project_amd.workloads import HEADLINE, PAIRS, check_traffic_sources, measured_traffic
    got = check_traffic_sources()
    assert len(got) == 5
    for n, (k1, k2, kind, suffix) in HEADLINE.items():
        t = got[f"{k1}_{k2}_fused_{kind}{suffix}"]
        alg = PAIRS[n].bytes1 + PAIRS[n].bytes2
        assert alg <= t <= 3 * alg, (n, t, alg)
    assert measured_traffic("bias_relu_4096") is None
