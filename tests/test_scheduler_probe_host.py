"""The statistics of the hardware-scheduler experiment (tests/interleave_scheduler/test/test_scheduler.py:77-131 of
the reference) over a placement that is written down here, no GPU: the MI355X dispatcher as the probe records it --
workgroup i on XCD i % 8, the j-th workgroup of an XCD on CU j % 32 of it."""
import numpy as np
import pytest

from bfuse_project_amd import scheduler_probe as sp
from bfuse_project_amd.patterns import LaunchDims, plan_blocks


def _round_robin(n):
    i = np.arange(n)
    return (i % 8) * 32 + (i // 8) % 32, i % 8       # CU, XCD


def _sides(pattern, grids, p0=1, p1=1):
    return plan_blocks(pattern, [LaunchDims((g, 1, 1), (256, 1, 1)) for g in grids], p0, p1).table()[0]


def test_one_to_one_interleave_parks_each_operator_on_four_xcds():
    side = _sides("zigzag", (2048, 2048))
    assert list(side[:6]) == [0, 1, 0, 1, 0, 1]
    cu, xcd = _round_robin(side.size)
    s = sp.mix_statistics(cu, side)
    assert s["units"] == 256 and s["mean_diff"] == 1.0 and s["max_share"] in ((1.0, 0.0), (0.0, 1.0))
    x = sp.mix_statistics(xcd, side)
    assert x["units"] == 8 and x["mean_diff"] == 1.0
    assert np.all(x["n0"][0::2] == 512) and np.all(x["n0"][1::2] == 0) and np.all(x["n1"][1::2] == 512)


def test_chunks_of_one_round_over_the_cus_mix_evenly():
    side = _sides("chunked", (2048, 2048), 256)
    cu, xcd = _round_robin(side.size)
    s = sp.mix_statistics(cu, side)
    assert s["mean_diff"] == 0.0 and s["max_share"] == (0.5, 0.5) and np.all(s["n0"] == 8) and np.all(s["n1"] == 8)
    assert sp.mix_statistics(xcd, side)["mean_diff"] == 0.0
    # the reference reads only the first 4000 lines of its log: a prefix that ends inside a chunk is uneven
    assert 0.0 < sp.mix_statistics(cu, side, first=4000)["mean_diff"] < 0.2


def test_statistics_by_hand():
    #           unit: 0  0  0  1  1  2
    s = sp.mix_statistics([0, 0, 0, 1, 1, 2], [0, 0, 1, 0, 1, 1])
    assert list(s["n0"]) == [2, 1, 0] and list(s["n1"]) == [1, 1, 1]
    assert s["max_unit"] == 0 and s["max_share"] == (2 / 3, 1 / 3)          # the first unit with the largest |n0 - n1|
    assert s["min_unit"] == 1 and s["min_share"] == (0.5, 0.5)
    assert s["mean_diff"] == pytest.approx((1 / 3 + 0 + 1) / 3)
    with pytest.raises(ValueError):
        sp.mix_statistics([0, 1], [0])
    # a unit that received nothing among the first ids is left out, as the reference skips its -1 entries
    assert sp.mix_statistics([0, 0, 5], [0, 1, 1], first=2)["units"] == 1


def test_arrival_map_and_cu_numbering():
    m = sp.arrival_map([0, 1, 0, 1, 0], [0, 1, 1, 0, 0], rows=70, color=False)
    assert m.splitlines() == ["01", "10", "0 "]
    assert sp.RED + "0" + sp.RESET in sp.arrival_map([0], [0])
    assert sp.arrival_map([0, 0, 0], [1, 1, 0], rows=2, color=False).splitlines() == ["1", "1"]
    idx = sp.cu_index(np.array([1, 0, 1, 0]), np.array([0, 3, 0, 3]), np.array([5, 7, 5, 6]))
    assert list(idx) == [2, 1, 2, 0]
