"""Pins the oracle's merge-path functions (oracle/mp_oracle.c) without a GPU.

The reference has no tests or golden vectors, so the literal restatement of
MergePathSearch / generate_mp_sched is pinned by: hand-worked coordinates
(tests/golden/worked_examples.json), a closed form, a brute-force merge walk
over every diagonal, the invariants of a merge path, and the tiling property
of the schedule.
"""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "worked_examples.json")


def random_row_ptr(rng, n, max_deg, p_empty=0.3):
    deg = rng.integers(0, max_deg + 1, size=n)
    deg[rng.random(n) < p_empty] = 0
    return np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)


@pytest.fixture(scope="module")
def golden():
    with open(GOLDEN) as f:
        return json.load(f)


def test_num_partitions_table(orc, golden):
    for row in golden["num_partitions"]:
        assert orc.num_partitions(row["n_rows"], row["nnz"], row["cost"]) == row["P"]


def test_worked_coordinates(orc, golden):
    for case in golden["coords"]:
        rp = np.array(case["row_ptr"], dtype=np.int32)
        xs, ys = orc.partition_coords(rp, int(rp[-1]), case["P"])
        assert xs.tolist() == case["x"]
        assert ys.tolist() == case["y"]


def test_worked_schedule(orc, golden):
    for case in golden["sched"]:
        rp = np.array(case["row_ptr"], dtype=np.int32)
        sched = orc.generate_mp_sched(rp, int(rp[-1]), case["P"])
        for name in orc.SCHED_FIELDS:
            assert sched[name].tolist() == case[name], name


def test_search_equals_closed_form_and_walk(orc):
    rng = np.random.default_rng(1234)
    for trial in range(300):
        n = int(rng.integers(0, 12))
        rp = random_row_ptr(rng, n, int(rng.integers(1, 9)))
        nnz = int(rp[-1])
        xs, ys = orc.merge_path_walk(rp, nnz)
        total = rp.size + nnz
        for d in range(total + 1):
            lit = orc.merge_path_search(d, rp, nnz)
            assert lit == orc.merge_path_closed_form(d, rp), (rp, d)
            assert lit == (int(xs[d]), int(ys[d])), (rp, d)


def test_path_invariants(orc):
    rng = np.random.default_rng(99)
    for trial in range(50):
        n = int(rng.integers(1, 200))
        rp = random_row_ptr(rng, n, 40)
        nnz = int(rp[-1])
        total = rp.size + nnz
        prev = (0, 0)
        for d in range(total + 1):
            x, y = orc.merge_path_search(d, rp, nnz)
            assert x + y == d
            assert (x == 0) == (d == 0)
            assert x >= prev[0] and y >= prev[1]
            if x >= 1:
                assert rp[x - 1] <= y
                assert y <= (rp[x] if x < rp.size else nnz)
            prev = (x, y)
        assert prev == (rp.size, nnz)


def covered_by_schedule(rp, sched, P):
    """Nonzeros the reference kernel would touch given the six arrays
    (src/MergePathSpMM.cu:435-477): head if fstart != 0, whole rows, tail if fend != 0."""
    nnz = int(rp[-1])
    cover = np.zeros(nnz, dtype=np.int64)
    lost = np.zeros(nnz, dtype=np.int64)
    for p in range(P):
        start, end = int(sched["start_row"][p]), int(sched["end_row"][p])
        fs, fsn = int(sched["feature_start"][p]), int(sched["feature_start_num"][p])
        fe, fen = int(sched["feature_end"][p]), int(sched["feature_end_num"][p])
        if fs != 0:
            cover[fs:fs + fsn] += 1
            start += 1
        for r in range(start, end):
            cover[rp[r]:rp[r + 1]] += 1
        if fe != 0:
            cover[fe:fe + fen] += 1
        elif fen != 0:
            lost[0:fen] += 1  # tail that starts at nonzero 0: encoded as "none"
    return cover, lost


def test_schedule_tiles_the_nonzeros(orc):
    rng = np.random.default_rng(7)
    for trial in range(120):
        n = int(rng.integers(1, 60))
        rp = random_row_ptr(rng, n, 30)
        nnz = int(rp[-1])
        P = int(rng.integers(1, 40))
        sched = orc.generate_mp_sched(rp, nnz, P)
        cover, lost = covered_by_schedule(rp, sched, P)
        assert cover.max(initial=0) <= 1
        # every nonzero is covered exactly once, except those of a tail whose
        # first nonzero has index 0 (the zero sentinel of :366-369, :467)
        assert np.array_equal(cover + lost, np.ones(nnz, dtype=np.int64))
        xs, ys = orc.partition_coords(rp, nnz, P)
        assert np.array_equal(sched["end_row"], xs[1:] - 1)
        assert np.array_equal(sched["start_row"], np.maximum(xs[:-1] - 1, 0))


def test_partitions_beyond_total(orc):
    rp = np.array([0, 3, 3, 4, 9], dtype=np.int32)
    xs, ys = orc.partition_coords(rp, 9, 40)  # P > N + 1 + nnz: ipt = 1, trailing partitions empty
    assert xs[-1] == rp.size and ys[-1] == 9
    assert (np.diff(xs) >= 0).all() and (np.diff(ys) >= 0).all()
    assert (xs[15:] == rp.size).all() and (ys[15:] == 9).all()


def test_rowwise_bounds_table(orc, golden):
    for case in golden["rowwise_bounds"]:
        s, e = orc.rowwise_bounds(case["n_rows"], case["num_warps"])
        assert s.tolist() == case["start"] and e.tolist() == case["end"]


def test_build_part(orc):
    rng = np.random.default_rng(5)
    rp = np.array([0, 5, 5, 6, 14, 15], dtype=np.int32)
    pp, pn = orc.build_part(4, rp)  # degrees 5,0,1,8,1 -> 2+0+1+2+1 groups
    assert pp.tolist() == [0, 4, 5, 6, 10, 14, 15]
    assert pn.tolist() == [0, 0, 2, 3, 3, 4]
    for trial in range(100):
        n = int(rng.integers(1, 80))
        rp = random_row_ptr(rng, n, 50)
        ps = int(rng.integers(1, 20))
        pp, pn = orc.build_part(ps, rp)
        deg = np.diff(rp)
        assert pn.size == orc.calculate_part_num(ps, rp) == int(np.sum((deg + ps - 1) // ps))
        assert pp[-1] == rp[-1]
        sizes = np.diff(pp)
        assert (sizes >= 1).all() and (sizes <= ps).all()
        assert (rp[pn] <= pp[:-1]).all() and (pp[1:] <= rp[pn + 1]).all()
