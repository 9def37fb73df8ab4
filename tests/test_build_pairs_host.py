"""build_pairs on the host: which fused kernels a suite lacks, the translation unit written for them, and the
registry's own spelling of the operator types (no GPU, nothing compiled here -- the build step compiles the
sample suite and the GPU tests run it)."""
import os
from types import SimpleNamespace as NS

import pytest
import yaml

import bfuse_project_amd as bf
from bfuse_project_amd import build_pairs, configure

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _k(name, threads, barriers, kind=0):
    return NS(name=name, block=(threads, 1, 1), has_barriers=barriers, kind=kind)


def test_wanted_skips_what_the_registry_holds_and_writes_thread_fusion_only_where_it_fits():
    reg = {k.name: k for k in (_k("a", 256, True), _k("b", 64, False), _k("c", 256, True), _k("d", 896, False),
                               _k("a_b_fused_bfuse_c256", 256, True, kind=1))}
    lds = {"a": 70000, "b": 0, "c": 100000, "d": 0}.__getitem__
    got = build_pairs.wanted([("a", "b"), ("a", "c"), ("a", "d"), ("c", "b"), ("a", "b")], reg, "both", 256, lds)
    names = [k["name"] for k in got]
    assert names == ["a_b_fused_hfuse",                                   # block-fused a+b is already there
                     "a_c_fused_bfuse_c256",                              # both sides synchronise: no thread-level fusion
                     "a_d_fused_bfuse_c256",                              # 256 + 896 threads do not fit one workgroup
                     "c_b_fused_bfuse_c256", "c_b_fused_hfuse"]
    assert [k["name"] for k in build_pairs.wanted([("c", "b")], reg, "bfuse", 128, lds)] == ["c_b_fused_bfuse_c128"]
    assert [k["name"] for k in build_pairs.wanted([("c", "b")], reg, "bfuse", 256, lds, rt=True)] == ["c_b_fused_bfuse_c256", "c_b_fused_bfuse_rt"]
    # LDS: 100000 + 70000 bytes exceed a workgroup's 160 KB
    reg["e"] = _k("e", 64, False)
    assert [k["form"] for k in build_pairs.wanted([("c", "e")], reg, "both", 256, {"c": 100000, "e": 70000}.__getitem__)] == ["bfuse"]
    with pytest.raises(LookupError):
        build_pairs.wanted([("a", "zz")], reg)
    with pytest.raises(LookupError):
        build_pairs.wanted([("a", "a_b_fused_bfuse_c256")], reg)


def test_source_text_names_each_side_once_by_the_type_the_library_gives():
    todo = [{"k1": "a", "k2": "b", "form": "bfuse", "name": "a_b_fused_bfuse_c256"},
            {"k1": "a", "k2": "b", "form": "hfuse", "name": "a_b_fused_hfuse"},
            {"k1": "c", "k2": "b", "form": "bfuse", "name": "c_b_fused_bfuse_c256"},
            {"k1": "c", "k2": "b", "form": "rt", "name": "c_b_fused_bfuse_rt"}]
    text = build_pairs.source_text(todo, 256, {"a": "bfuse::A<1, 2>", "b": "bfuse::B<true>", "c": "bfuse::C<3>"}.__getitem__)
    lines = text.splitlines()
    assert lines.count("using Side0 = bfuse::A<1, 2>;   // a") == 1 and "using Side1 = bfuse::B<true>;   // b" in lines
    assert "BFUSE_BFUSE_KERNEL(a, Side0, b, Side1, _c256, bfuse::kChunked, 256, 1)" in lines
    assert "BFUSE_HFUSE_KERNEL(a, Side0, b, Side1)" in lines
    assert "BFUSE_BFUSE_KERNEL(c, Side2, b, Side1, _c256, bfuse::kChunked, 256, 1)" in lines
    assert "BFUSE_BFUSE_RT_KERNEL(c, Side2, b, Side1)" in lines
    assert [build_pairs._unit_kernel(l) for l in lines if l.startswith("BFUSE_")][-4:] == [k["name"] for k in todo]
    assert "BFUSE_MODULE_PROLOGUE()" in lines and '#include "fuse.h"' in lines
    for h in build_pairs.HEADERS:
        assert os.path.exists(os.path.join(build_pairs.CSRC, h))


def test_registry_spells_operator_types_and_their_lds():
    assert build_pairs.op_type("gemm_f32_512x768x2304") == "bfuse::GemmF32Dma<512, 2304, 768, 32, 144, 4>"
    assert build_pairs.op_type("conv3x3s1p1_f32_1024x448x8x8_384").startswith("bfuse::ConvF32Lds<448, 384, 8, 8, 3, 3, 1, 1,")
    assert build_pairs.op_type("conv1x1s1p0_f32_64x56x56_64") == "bfuse::SwapOperands<bfuse::GemmF32<64, 3136, 64, 16, 64, 1>>"
    assert build_pairs.op_lds("gemm_f32_512x768x2304") == 73728        # four waves x three stages of 6 KB
    assert build_pairs.op_lds("layernorm_512x768") >= 0
    with pytest.raises(LookupError):
        build_pairs.op_type("gemm_f32_512x768x2304_layernorm_512x768_fused_bfuse_r")    # a fused kernel has no operator type
    assert build_pairs.op_lds("no_such_kernel") == -1
    # every standalone kernel has a type that names a template of the library
    for k in bf.list_kernels():
        if k.kind == 0:
            assert build_pairs.op_type(k.name).startswith("bfuse::"), k.name


def test_sample_suite_lists_six_kernels_to_build(tmp_path):
    """The example the build step compiles: four pairs, none with a fused kernel in the library; both forms where
    thread-level fusion fits (the one-wave batched product beside a convolution), block fusion alone for the
    four-wave dense layer beside a four-wave convolution (both synchronise)."""
    out = tmp_path / "s"
    r = configure.configure(os.path.join(ROOT, "bfuse-project_amd", "examples", "batch_operators.yaml"), str(out))
    assert not r["missing"] and all(not v for v in r["fused"].values())
    b = build_pairs.build(str(out), compile_=False)
    assert sorted(k["form"] for k in b["kernels"]) == ["bfuse"] * 4 + ["hfuse"] * 2
    assert len(b["files"]) == 3 and all(os.path.exists(f) for f in b["files"])
    assert build_pairs.module_paths(str(out)) == []          # nothing compiled, nothing to load
    with pytest.raises(LookupError):
        build_pairs.build(str(out), only=["a+b"], compile_=False)
    with open(out / "config" / "modules.yaml", "w") as f:
        yaml.safe_dump(["hip/libbfuse_pairs.so"], f)
    assert build_pairs.module_paths(str(out)) == [os.path.join(str(out), "hip", "libbfuse_pairs.so")]


def test_units_written_for_another_tiling_of_an_operator_are_found(tmp_path):
    """A suite's translation units name each side by the operator type the library gave it when they were written;
    after a rebuild of the library with another tiling they are stale and must be written again."""
    d = tmp_path / "hip"
    d.mkdir()
    (d / "pairs_0.hip").write_text("using Side0 = bfuse::A<1>;   // a\nusing Side1 = bfuse::B<2>;   // b\nBFUSE_HFUSE_KERNEL(a, Side0, b, Side1)\n")
    (d / "pairs_1.hip").write_text("using Side0 = bfuse::A<1>;   // a\nBFUSE_HFUSE_KERNEL(a, Side0, a, Side0)\n")
    now = {"a": "bfuse::A<1>", "b": "bfuse::B<3>"}.__getitem__
    assert build_pairs.stale_units(str(d), now) == ["pairs_0.hip"]
    assert build_pairs.stale_units(str(d), {"a": "bfuse::A<1>", "b": "bfuse::B<2>"}.__getitem__) == []
    assert build_pairs.stale_units(str(tmp_path / "none")) == []
