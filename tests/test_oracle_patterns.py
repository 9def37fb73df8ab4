"""Pins the index-map oracle (oracle/patterns_ref.c) against the reference's own emitted
prologues and YAML outputs (fixtures under tests/golden/, made by make_pattern_goldens.py),
and against what the mathematics fixes (bijection onto the disjoint union of the grids)."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as ork


def _load(golden_dir, name):
    return json.load(open(os.path.join(golden_dir, name)))


def _gs(grids):
    return [g[0] * g[1] * g[2] for g in grids]


def test_fused_dims_match_reference_yaml(golden_dir):
    data = _load(golden_dir, "fused_dims.json")
    assert data["rows_read"] >= 2728
    for row in data["unique"]:
        g1, t1, g2, t2 = row["k"]
        fg, fb = ork.bfuse_dims([g1, g2], [t1, t2])
        assert [fg, 1, 1] == row["bfuse"][0] and [fb, 1, 1] == row["bfuse"][1]
        lo, hi, hg, hb = ork.hfuse_dims([g1, g2], [t1, t2], pad=32)
        assert [hg, 1, 1] == row["hfuse"][0] and [hb, 1, 1] == row["hfuse"][1]


def test_bfuse_maps_match_emitted_prologues(golden_dir):
    recs = _load(golden_dir, "bfuse_maps.json")
    kinds = set()
    for r in recs:
        gs = _gs(r["grids"])
        if r["pattern"] == "zigzag":
            k, v = ork.map_table("zigzag", gs, r["params"]["M"], r["params"]["N"])
        else:
            k, v = ork.map_table("chunk", gs, r["params"]["TotalSM"])
        kinds.add((r["pattern"], tuple(sorted(r["params"].items()))))
        fg, fb = ork.bfuse_dims(r["grids"], r["blocks"])
        assert fg == r["fused_grid"] and fb == r["fused_block"], r["source"]
        s = np.array(r["samples"])
        assert np.array_equal(k[s[:, 0]], s[:, 1]), r["source"]
        assert np.array_equal(v[s[:, 0]], s[:, 2]), r["source"]
    # the fixtures cover 1:1, several M:1 and N:N ratios, and the SM-chunk pattern
    assert ("chunk", (("TotalSM", 84),)) in kinds
    assert len([k for k in kinds if k[0] == "zigzag"]) >= 10


def test_hfuse_ranges_match_emitted_guards(golden_dir):
    for r in _load(golden_dir, "hfuse_ranges.json"):
        grids = [[s["grid_xy"][0], s["grid_xy"][1], s["blocks"] // s["grid_xy"][2]] for s in r["sides"]]
        nthreads = [s["thr_hi"] - s["thr_lo"] for s in r["sides"]]
        blocks = [[s["block_xy"][0], s["block_xy"][1], nt // s["block_xy"][2]] for s, nt in zip(r["sides"], nthreads)]
        lo, hi, fg, fb = ork.hfuse_dims(grids, blocks, pad=32)
        assert lo == [s["thr_lo"] for s in r["sides"]], r["source"]
        assert hi == [s["thr_hi"] for s in r["sides"]], r["source"]
        assert fb == r["fused_block"]
        assert fg == max(s["blocks"] for s in r["sides"])
        # bar.sync <side+1>, <pad32(T)>  (Matchers.cc:288-320)
        want = sorted([i + 1, -(-nt // 32) * 32] for i, nt in enumerate(nthreads))
        assert r["barriers"] == want, r["source"]
        # remap of one thread per side
        for i, s in enumerate(r["sides"]):
            bid, tid = s["blocks"] - 1, s["thr_hi"] - 1
            k, vb, vt = ork.hfuse_map(grids, blocks, 32, bid, tid)
            assert k == i
            g, b = grids[i], blocks[i]
            assert vb[0] + g[0] * (vb[1] + g[1] * vb[2]) == bid
            assert vt[0] + b[0] * (vt[1] + b[1] * vt[2]) == tid - s["thr_lo"]
        # a thread in the padding gap, or a block past a side's grid, belongs to nobody
        if r["sides"][0]["thr_hi"] < r["sides"][1]["thr_lo"]:
            assert ork.hfuse_map(grids, blocks, 32, 0, r["sides"][0]["thr_hi"])[0] == -1
        small = min(range(2), key=lambda i: r["sides"][i]["blocks"])
        if r["sides"][small]["blocks"] < fg:
            assert ork.hfuse_map(grids, blocks, 32, fg - 1, r["sides"][small]["thr_lo"])[0] == -1


def _assert_bijection(k, v, gs):
    assert k.min() >= 0
    for i, g in enumerate(gs):
        vv = np.sort(v[k == i])
        assert np.array_equal(vv, np.arange(g)), (i, g)


@pytest.mark.parametrize("kind,params", [
    ("zigzag", (1, 1)), ("zigzag", (2, 1)), ("zigzag", (4, 3)), ("zigzag", (1, 5)), ("zigzag", (64, 1)),
    ("prop", (1, 1)), ("prop", (3, 1)), ("prop", (1000, 1)),
    ("chunk", (1, 1)), ("chunk", (8, 1)), ("chunk", (84, 1)), ("chunk", (256, 1)),
])
def test_maps_are_bijections(kind, params):
    rng = np.random.default_rng(3)
    cases = [(1, 1), (1, 7), (7, 1), (5, 5), (256, 128), (288, 128), (3, 1000), (1000, 3), (84, 84), (85, 167)]
    cases += [tuple(int(x) for x in rng.integers(1, 700, 2)) for _ in range(60)]
    for gs in cases:
        k, v = ork.map_table(kind, gs, *params)
        _assert_bijection(k, v, gs)
        # one past the end matches no branch
        k2, _ = ork.map_table(kind, gs, *params, lo=sum(gs), hi=sum(gs) + 1)
        assert k2[0] == -1


def test_three_kernels_ratio_maps_are_bijections():
    rng = np.random.default_rng(11)
    for _ in range(40):
        gs = [int(x) for x in rng.integers(1, 300, 3)]
        for kind, params in (("zigzag", (1, 1)), ("zigzag", (3, 2)), ("prop", (1, 1))):
            k, v = ork.map_table(kind, gs, *params)
            _assert_bijection(k, v, gs)


def test_prop_reduces_to_zigzag():
    """coarseInterleaveWithoutSMPattern with MinOption=1 uses ratio floor(g_k/g_min); the live
    pattern gives the same ratios when M exceeds every ratio and N=1, so the tables agree."""
    rng = np.random.default_rng(5)
    for _ in range(50):
        gs = [int(x) for x in rng.integers(1, 900, 2)]
        M = max(gs) // min(gs) + 1
        k1, v1 = ork.map_table("prop", gs, 1)
        k2, v2 = ork.map_table("zigzag", gs, M, 1)
        assert np.array_equal(k1, k2) and np.array_equal(v1, v2)


def test_zigzag_1to1_closed_form():
    """M=N=1: even ids -> kernel 0, odd -> kernel 1 until the smaller grid is used up, then the
    rest of the larger grid in order."""
    for gs in [(384, 100352), (7, 3), (10, 10), (1, 9)]:
        k, v = ork.map_table("zigzag", gs, 1, 1)
        m = min(gs)
        assert np.array_equal(k[: 2 * m], np.tile([0, 1], m))
        assert np.array_equal(v[: 2 * m], np.repeat(np.arange(m), 2))
        big = int(np.argmax(gs)) if gs[0] != gs[1] else None
        if big is not None:
            assert np.all(k[2 * m:] == big)
            assert np.array_equal(v[2 * m:], np.arange(m, gs[big]))


def test_chunk_pattern_alternates_whole_chunks():
    gs, sm = (1024, 1815), 84
    k, v = ork.map_table("chunk", gs, sm)
    # first region: 12 rounds of [84 of kernel 0][84 of kernel 1]
    assert np.array_equal(k[:2016].reshape(12, 2, 84), np.broadcast_to(np.array([0, 1])[None, :, None], (12, 2, 84)))
    assert np.all(k[2016:2772] == 1) and np.all(k[2772:2788] == 0) and np.all(k[2788:] == 1)


def test_virtual_ids_roundtrip():
    grid, block = [55, 11, 3], [19, 1, 8]
    for nb in (0, 54, 55, 604, 605, 1814):
        for tid in (0, 18, 19, 151):
            vb, vt = ork.virtual_ids(grid, block, nb, tid)
            assert vb[0] + grid[0] * (vb[1] + grid[1] * vb[2]) == nb
            assert vt[0] + block[0] * (vt[1] + block[1] * vt[2]) == tid
            assert all(0 <= a < b for a, b in zip(vb, grid)) and all(0 <= a < b for a, b in zip(vt, block))


def test_check_matrix_rule():
    a = np.array([0.0, 1.0, 1000.0, 1e-6, 5.0], np.float32)
    o = np.array([0.0005, 1.0005, 1000.5, 0.002, 5.1], np.float32)
    #           abs ok   abs ok   rel ok    fails   fails
    assert ork.check_matrix(o, a, 1e-3) == 2
    assert ork.check_matrix(a, a, 1e-3) == 0
    o2 = a.copy(); o2[0] = 0.002   # a == 0 and abs error above eps -> wrong
    assert ork.check_matrix(o2, a, 1e-3) == 1


def _prop_table_min_option(min_option):
    """coarseInterleaveWithoutSMPattern for grids (10, 26), worked by hand from Algorithms.cc:323-355.

    MinOption = 2: MinRatio = 10 / 2 = 5; ratios 10/5 = 2 and 26/5 = 5; quotients 10/2 = 5 and 26/5 = 5,
    MinQuot = 5; rotation 7 = [k0 k0 k1 k1 k1 k1 k1]; interleaved region 7 * 5 = 35 ids; remainders
    10 - 10 = 0 and 26 - 25 = 1, so id 35 is kernel 1's block 25.
    MinOption = 3: MinRatio = 10 / 3 = 3; ratios 10/3 = 3 and 26/3 = 8; quotients 10/3 = 3 and 26/8 = 3,
    MinQuot = 3; rotation 11 = [k0 x3, k1 x8]; region 33 ids; remainders 10 - 9 = 1 (id 33 -> kernel 0
    block 9) and 26 - 24 = 2 (ids 34, 35 -> kernel 1 blocks 24, 25)."""
    if min_option == 2:
        rows = [
            [(0, 0), (0, 1), (1, 0), (1, 1), (1, 2), (1, 3), (1, 4)],
            [(0, 2), (0, 3), (1, 5), (1, 6), (1, 7), (1, 8), (1, 9)],
            [(0, 4), (0, 5), (1, 10), (1, 11), (1, 12), (1, 13), (1, 14)],
            [(0, 6), (0, 7), (1, 15), (1, 16), (1, 17), (1, 18), (1, 19)],
            [(0, 8), (0, 9), (1, 20), (1, 21), (1, 22), (1, 23), (1, 24)],
            [(1, 25)],
        ]
    else:
        rows = [
            [(0, 0), (0, 1), (0, 2), (1, 0), (1, 1), (1, 2), (1, 3), (1, 4), (1, 5), (1, 6), (1, 7)],
            [(0, 3), (0, 4), (0, 5), (1, 8), (1, 9), (1, 10), (1, 11), (1, 12), (1, 13), (1, 14), (1, 15)],
            [(0, 6), (0, 7), (0, 8), (1, 16), (1, 17), (1, 18), (1, 19), (1, 20), (1, 21), (1, 22), (1, 23)],
            [(0, 9), (1, 24), (1, 25)],
        ]
    flat = [kv for row in rows for kv in row]
    return np.array([k for k, _ in flat]), np.array([v for _, v in flat])


@pytest.mark.parametrize("min_option", [2, 3])
def test_prop_map_with_min_option_against_a_hand_worked_table(min_option):
    """The reference never emitted this pattern (dead code, Contexts.cc:77-78), so no golden exists
    for MinOption > 1; a table worked by hand from the source pins the divisor and the remainders
    (with MinOption ignored the rotation would be [k0, k1, k1] and the table differs from id 1 on)."""
    k_want, v_want = _prop_table_min_option(min_option)
    k, v = ork.map_table("prop", (10, 26), min_option)
    assert k.size == 36 and np.array_equal(k, k_want) and np.array_equal(v, v_want)
    k1, v1 = ork.map_table("prop", (10, 26), 1)
    assert not np.array_equal(k1, k_want)
    # the product's host map (csrc/dispatch.h through the C ABI) against the same table
    import bfuse_project_amd as bf
    plan = bf.plan_blocks("proportional", [bf.LaunchDims((10, 1, 1), (64, 1, 1)), bf.LaunchDims((26, 1, 1), (64, 1, 1))], min_option, 1)
    kp, vp = plan.table()
    assert plan.fused_grid == 36 and np.array_equal(kp, k_want) and np.array_equal(vp, v_want)
