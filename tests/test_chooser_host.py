"""The pattern chooser against the headline table (host logic: launch shapes and barrier flags
come from the registry without a GPU; register and LDS figures need one and are covered by the
GPU tests).

The reference hard-codes pattern and ratio (horizontal-fuser/src/Contexts.cc:64-79) and parses
Reg / HasBarriers without using them; here the fused kernel that is measured for each pair must be
the one the chooser selects.
"""
import os

import pytest

import bfuse_project_amd as bf
from bfuse_project_amd import config, patterns, tuner
from bfuse_project_amd.workloads import CONFIG_KINDS, GROUPS, HEADLINE, PAIRS


@pytest.mark.parametrize("number", sorted(PAIRS))
def test_static_choice_selects_the_headline_kernel(number):
    k1, k2, kind, suffix = HEADLINE[number]
    a, b = bf.kernel_info(k1), bf.kernel_info(k2)
    choice = tuner.static_plan(a, b, kinds=CONFIG_KINDS[number])
    assert choice["kind"] == kind
    h = tuner.find_variant(a, b, choice)
    assert h is not None and h.name == f"{k1}_{k2}_fused_{kind}{suffix}"


@pytest.mark.parametrize("group", sorted(GROUPS))
def test_static_choice_of_a_group_selects_the_measured_kernel(group):
    names, kind, suffixes, _ = GROUPS[group]
    ks = [bf.kernel_info(n) for n in names]
    choice = tuner.static_plan_group(ks)
    assert choice["kind"] == kind == "bfuse" and (choice["pattern"], choice["p0"]) == ("chunked", 256)
    h = tuner.find_group_variant(ks, choice)
    assert h is not None and h.name == "_".join(names) + f"_fused_{kind}{suffixes[0]}" and h.n_sides == len(names)
    # a plan nobody built resolves to nothing
    assert tuner.find_group_variant(ks, {"kind": "bfuse", "pattern": "zigzag", "p0": 3, "p1": 2}) is None


def test_plans_of_different_patterns_can_coincide_and_are_recognised():
    d = [patterns.LaunchDims((196, 1, 1), (256, 1, 1)), patterns.LaunchDims((196, 1, 1), (256, 1, 1))]
    assert tuner.same_dispatch(patterns.plan_blocks("chunked", d, 256, 1), patterns.plan_blocks("ranges", d, 1, 1))
    assert not tuner.same_dispatch(patterns.plan_blocks("chunked", d, 8, 1), patterns.plan_blocks("ranges", d, 1, 1))
    d2 = [patterns.LaunchDims((256, 1, 1), (256, 1, 1)), patterns.LaunchDims((512, 1, 1), (64, 1, 1))]
    assert tuner.same_dispatch(patterns.plan_blocks("chunked", d2, 256, 1), patterns.plan_blocks("ranges", d2, 1, 1))


def test_footprint_rules():
    def ki(name, barriers, grid, threads, regs):
        return config.KernelInfo(name, barriers, (grid, 1, 1), (threads, 1, 1), regs)
    # barriers on both sides: block fusion, whatever else holds
    c = config.choose_fusion(ki("a", True, 256, 256, 64), ki("b", True, 256, 256, 64), 1024, 1024)
    assert not c["hfuse_ok"] and c["prefer"] == "bfuse"
    # matching grids, one barrier-free side: thread-level fusion
    c = config.choose_fusion(ki("a", True, 256, 128, 64), ki("b", False, 256, 128, 32), 4096, 0)
    assert c["hfuse_ok"] and c["prefer"] == "hfuse"
    # summed LDS beyond a CU's 160 KB: block fusion
    c = config.choose_fusion(ki("a", True, 256, 128, 64), ki("b", False, 256, 128, 32), 100 * 1024, 70 * 1024)
    assert not c["hfuse_ok"]
    # workgroups per CU follow the larger side's registers and LDS (a fused kernel allocates both for every workgroup)
    c = config.choose_fusion(ki("a", True, 512, 256, 94), ki("b", False, 1536, 256, 40), 32 * 1024, 0)
    assert c["wg_per_cu"] == (5, 5) and c["chunk"] == 256
    c = config.choose_fusion(ki("a", True, 256, 768, 168), ki("b", False, 512, 64, 48), 135 * 1024, 0)
    assert c["wg_per_cu"][0] == 1 and c["wg_per_cu"][1] == 1      # 135 KB: nothing shares the CU with it


def test_the_footprint_rule_on_the_48_pairs_of_the_model_operator_matrix(golden_dir):
    """Footprints of the library's own kernels (registers and LDS from the build's resource remarks, launch
    shapes from the registry) and one measured run of the 48-pair matrix (standalone times, speed-up of the
    block-fused kernel over serial; tests/golden/model_matrix_footprints.json).  The rule sees footprints and
    standalone times only.  It must leave unfused every pair whose block-fused kernel measured slower than
    serial, fuse at least half of the pairs that gained 5 % or more, and its choices must come out ahead."""
    import json
    import math
    import os
    with open(os.path.join(golden_dir, "model_matrix_footprints.json")) as f:
        data = json.load(f)

    def ki(name):
        k = data["kernels"][name]
        return config.KernelInfo(name, k["barriers"], (k["grid"], 1, 1), (k["threads"], 1, 1), k["regs"], k["us"]), k["lds"]

    assert len(data["pairs"]) == 48
    log_gain, fused, missed = 0.0, 0, 0
    for p in data["pairs"]:
        (a, la), (b, lb) = ki(p["kernel1"]), ki(p["kernel2"])
        c = config.choose_fusion(a, b, la, lb, matrix=(True, True))    # GEMMs, batched products, convolutions
        assert c["fuse"] in ("bfuse", "none")            # no pair of the matrix has matching grids
        if p["bfuse_speedup"] < 0.98:
            assert c["fuse"] == "none", (p, c)
        if c["fuse"] == "bfuse":
            assert p["bfuse_speedup"] >= 0.98, (p, c)
            log_gain += math.log(p["bfuse_speedup"])
            fused += 1
        elif p["bfuse_speedup"] >= 1.05:
            missed += 1
        assert c["fuse"] == p["chooser"]                 # what the suite's run decided on the GPU box
    winners = sum(1 for p in data["pairs"] if p["bfuse_speedup"] >= 1.05)
    assert fused >= 20 and missed <= winners // 2
    assert math.exp(log_gain / 48) >= 1.04


def test_the_footprint_rule_on_the_headline_pairs_with_and_without_times():
    """Pairs 2 and 4: the memory-bound side does not fit a CU next to the GEMM in one round, but its workgroups
    are short (a row each) and end in the GEMM's shadow: block fusion pays.  A batched GEMM whose workgroups
    live as long as the kernel does not.  Without times, only a side with neither barriers nor LDS is taken
    for short-lived."""
    ki = config.KernelInfo
    gemm2 = ki("gemm_f32_512x768x2304", True, (256, 1, 1), (256, 1, 1), 156, 15.6)
    ln = ki("layernorm_512x768", False, (512, 1, 1), (64, 1, 1), 46, 4.1)
    c = config.choose_fusion(gemm2, ln, 73728, 0)
    assert not c["side_by_side"] and c["bfuse_pays"] and c["fuse"] == "bfuse" and c["predicted_us"] == 15.6
    softmax = ki("softmax_causal_12x512x512", False, (1536, 1, 1), (256, 1, 1), 15, 5.2)
    gemm4 = ki("gemm_gelu_f32_512x768x3072", True, (512, 1, 1), (256, 1, 1), 90, 20.8)
    c = config.choose_fusion(softmax, gemm4, 0, 32768)
    assert not c["side_by_side"] and c["fuse"] == "bfuse"
    long_b = ki("bgemm_f32_32x512x512x128", True, (1024, 1, 1), (128, 1, 1), 100, 27.2)
    c = config.choose_fusion(ki("gemm_f32_512x768x768", True, (256, 1, 1), (256, 1, 1), 53, 7.0), long_b, 36864, 16384)
    assert c["fuse"] == "none" and c["predicted_us"] >= c["serial_us"]
    # no times: the LayerNorm (no barriers, no LDS) is taken for short-lived, the batched GEMM is not
    untimed = lambda k: ki(k.KernelName, k.HasBarriers, k.GridDim, k.BlockDim, k.Reg)
    assert config.choose_fusion(untimed(gemm2), untimed(ln), 73728, 0)["fuse"] == "bfuse"
    assert config.choose_fusion(ki("g", True, (256, 1, 1), (256, 1, 1), 53), untimed(long_b), 36864, 16384)["fuse"] == "none"
    # the bf16 gate projection's 135 KB leave room for nothing beside it: block fusion never pays, thread-level
    # fusion does when the grids match (pair 5)
    gate = ki("gemm_bf16_512x4096x14336", True, (256, 1, 1), (640, 1, 1), 116, 46.0)
    norm = ki("rmsnorm_rope_bf16_512x4096_w2", False, (256, 1, 1), (128, 1, 1), 60, 4.5)
    c = config.choose_fusion(gate, norm, 135168, 0)
    assert c["fuse"] == "hfuse" and not c["bfuse_pays"]
    assert tuner.static_plan.__defaults__[1] == ("hfuse", "bfuse")      # "none" is an answer only where it is asked for


def test_two_kernels_that_each_keep_every_matrix_pipe_busy_are_left_unfused():
    """The reference's benchmark arrangement (every dense layer, batched product and convolution at batch 1024
    against every other: bfuse-project_amd/examples/benchmark_batch1024.yaml, 903 pairs): measured on MI355X,
    block fusion 0.88x, thread-level fusion 0.63x of the two kernels one after the other -- each kernel already
    has a wave on every SIMD for its whole run.  The rule leaves every such pair unfused, from the registry's
    metadata alone; a matrix-core kernel that does not cover the chip (196 workgroups of a batch-1 convolution)
    or a side that is not a matrix-core kernel keeps the decision the footprints give."""
    import yaml
    import bfuse_project_amd as bf
    from bfuse_project_amd import configure, tuner
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "bfuse-project_amd", "examples", "benchmark_batch1024.yaml")) as f:
        doc = yaml.safe_load(f)
    registry = {k.name: k for k in bf.list_kernels()}
    found, missing = configure.resolve(doc, registry)
    assert not missing
    s0, s1 = (s["Set"] for s in doc["FusionSet"])
    n = 0
    for i, ka in enumerate(s0):
        for kb in s1[i:]:
            a, b = found[ka], found[kb]
            assert a.matrix and b.matrix
            c = tuner.static_plan(a, b, kinds=("hfuse", "bfuse", "none"), times=(100.0, 100.0))
            assert c["kind"] == "none" and c["static"]["saturates_matrix_cores"] == (True, True), (a.name, b.name)
            n += 1
    assert n == 903
    # same footprints, but the second side covers 196 of the 256 CUs: the matrix rule does not apply
    g = config.KernelInfo("g", True, (256, 1, 1), (256, 1, 1), 53, 7.0)
    conv = config.KernelInfo("c", True, (196, 1, 1), (256, 1, 1), 96, 7.2)
    assert config.choose_fusion(g, conv, 36864, 40000, matrix=(True, True))["fuse"] == config.choose_fusion(g, conv, 36864, 40000)["fuse"] == "bfuse"
    big = config.KernelInfo("c", True, (4096, 1, 1), (256, 1, 1), 96, 70.0)
    assert config.choose_fusion(g, big, 36864, 40000, matrix=(True, True))["fuse"] == "none"
    assert not bf.kernel_info("layernorm_512x768").matrix and bf.kernel_info("gemm_bf16_512x4096x14336").matrix
