"""The pattern chooser against the headline table (host logic: launch shapes and barrier flags
come from the registry without a GPU; register and LDS figures need one and are covered by the
GPU tests).

The reference hard-codes pattern and ratio (horizontal-fuser/src/Contexts.cc:64-79) and parses
Reg / HasBarriers without using them; here the fused kernel that is measured for each pair must be
the one the chooser selects.
"""
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
