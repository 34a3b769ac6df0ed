"""Sweep plans on the GPU, through the C ABI: parity with the fp64 CPU loop (the oracle), bit-identical repeats,
value refresh, edge shapes, both element types and every lane-group width."""
import numpy as np
import pytest
import torch

from tests.gpu_util import check_fp16, check_fp32, make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu

CASES = [
    # n, max_deg, hubs, K, dtype, piece, acc_rows, panels_per_round
    (300, 40, ((5, 280), (150, 300)), 16, "f32", 0, 0, 4),
    (97, 12, (), 32, "f32", 4, 0, 2),
    (513, 60, ((0, 500), (512, 400)), 64, "f32", 8, 64, 8),     # two column tiles, several rounds of panels
    (200, 5, (), 16, "f32", 2, 16, 256),                           # more panels than rows
    (5000, 200, ((17, 4800), (4999, 3000)), 128, "f32", 0, 0, 64),  # four column tiles; rows cut across panels
    (20000, 64, ((0, 15000),), 16, "f32", 0, 0, 0),
    (4096, 8, ((7, 4000), (2000, 3500)), 256, "f32", 0, 0, 16),
    (3000, 30, ((11, 2500),), 64, "f16", 0, 0, 8),                 # fp16, 128-byte rows: two accumulator planes
    (1000, 20, (), 32, "f16", 0, 0, 4),                            # fp16, 64-byte rows
    (700, 25, ((3, 650),), 128, "f16", 16, 0, 4),                  # fp16, two column tiles
    (1, 1, (), 16, "f32", 0, 0, 1),
    (3000, 40, ((5, 2800),), 16, "f32", 0, 0, 8, 2),               # 64-byte rows with pairs of instructions added up together
    (3000, 40, ((5, 2800),), 32, "f32", 0, 0, 8, 1),               # 128-byte rows, one instruction at a time
    (2000, 30, ((11, 1500),), 64, "f16", 0, 0, 8, 1),
    # rows of X that do not fill whole tiles: lanes past the row's end, lanes that straddle it, rows that start
    # between two 16-byte boundaries
    (300, 40, ((5, 280),), 8, "f32", 0, 0, 4),                     # 32-byte rows: half of the 4 lanes idle
    (500, 30, ((7, 450),), 12, "f32", 0, 0, 4),
    (400, 25, ((3, 390), (399, 380)), 20, "f32", 0, 0, 4),         # 80 bytes of a 128-byte tile
    (1000, 30, ((999, 900),), 24, "f32", 4, 0, 8),
    (600, 35, ((0, 550), (599, 500)), 41, "f32", 0, 0, 8),         # 164-byte rows: two tiles, the last lane straddles the end
    (800, 20, ((5, 700),), 48, "f32", 0, 0, 4, 2),
    (3000, 60, ((17, 2800), (2999, 2000)), 100, "f32", 0, 0, 64),  # four tiles, the last of them 16 bytes; rows cut across panels
    (200, 15, ((199, 190),), 7, "f32", 0, 0, 2),
    (150, 10, ((149, 140),), 1, "f32", 0, 0, 2),                   # one float per row
    (350, 22, ((349, 300),), 33, "f32", 0, 0, 4),
    (5000, 100, ((4999, 4500),), 200, "f32", 0, 0, 64),
    (400, 30, ((399, 350),), 8, "f16", 0, 0, 4),                   # 16-byte rows of halves
    (500, 30, ((499, 450),), 24, "f16", 0, 0, 4),
    (600, 30, ((599, 500),), 40, "f16", 0, 0, 8),                  # 80-byte rows: a 128-byte tile, two planes
    (700, 30, ((699, 600), (0, 650)), 72, "f16", 0, 0, 8),         # 144 bytes: two tiles
    (300, 20, ((299, 250),), 2, "f16", 0, 0, 2),                   # one dword per row
    (450, 25, ((449, 400),), 6, "f16", 0, 0, 4),
    (2500, 50, ((2499, 2300),), 100, "f16", 0, 0, 32),
]


def make_inputs(rng, n, max_deg, hubs, K, dt):
    rp, ci = random_csr(rng, n, max_deg, p_empty=0.25, hub_rows=hubs)
    npdt = np.float32 if dt == "f32" else np.float16
    val = rng.random(ci.size).astype(npdt)
    X = (rng.random((n, K)) * 2 - 1).astype(npdt)
    return rp, ci, val, X


@pytest.mark.parametrize("case", CASES)
def test_sweep_plan_matches_fp64_loop(pkg, orc, dev, case):
    n, max_deg, hubs, K, dt, piece, acc_rows, per_round = case[:8]
    together = case[8] if len(case) > 8 else 0
    rng = np.random.default_rng(abs(hash(case)) % (2 ** 32))
    rp, ci, val, X = make_inputs(rng, n, max_deg, hubs, K, dt)
    csr = make_csr(pkg, dev, rp, ci, val)
    # X between NaNs: what a lane reads past the end of a row must not reach a sum that is written out
    guard = 64
    xbuf = torch.full((n * K + 2 * guard,), float("nan"), dtype=torch.float32 if dt == "f32" else torch.float16, device=dev)
    d_X = xbuf[guard:guard + n * K].view(n, K)
    d_X.copy_(torch.from_numpy(X))
    plan = pkg.spmm.Plan(csr, K, sweep="force", sweep_piece=piece, sweep_acc_rows=acc_rows, sweep_panels_per_round=per_round,
                         sweep_together=together)
    i = plan.info
    assert i.sweep_panels > 0 and i.rowblock_steps == 0
    tile_bytes = i.sweep_lanes * 16
    assert (i.sweep_tiles - 1) * tile_bytes < K * X.itemsize <= i.sweep_tiles * tile_bytes
    # Y in the middle of a buffer of NaNs: nothing is written before its first or after its last element
    buf = torch.full((n * K + 2 * guard,), float("nan"), dtype=d_X.dtype, device=dev)
    Y = buf[guard:guard + n * K].view(n, K)
    plan.spmm(d_X, out=Y)
    torch.cuda.synchronize()
    assert torch.isnan(buf[:guard]).all() and torch.isnan(buf[guard + n * K:]).all()
    if dt == "f32":
        ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    else:
        ref, scale = orc.spmm_f64_f16in(rp, ci, val, X, want_abs=True)
        check_fp16(Y.cpu().numpy(), ref, scale)
    # repeats give the same bits, whatever Y held
    Y2 = torch.zeros_like(d_X)
    for _ in range(3):
        plan.spmm(d_X, out=Y2)
    torch.cuda.synchronize()
    assert torch.equal(Y, Y2)


def test_sweep_plan_closed_forms(pkg, dev):
    # identity: Y = X; all-ones features: row sums
    n = 1000
    rp = np.arange(n + 1, dtype=np.int32)
    ci = np.arange(n, dtype=np.int32)
    val = np.ones(n, dtype=np.float32)
    rng = np.random.default_rng(1)
    for K in (16, 32, 64):
        X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
        csr = make_csr(pkg, dev, rp, ci, val)
        (d_X,) = to_dev(dev, X)
        plan = pkg.spmm.Plan(csr, K, sweep="force", sweep_panels_per_round=8)
        assert np.array_equal(plan.spmm(d_X).cpu().numpy(), X)
    rp2, ci2 = random_csr(rng, n, 50, hub_rows=((3, 900),))
    v2 = rng.random(ci2.size).astype(np.float32)
    csr2 = make_csr(pkg, dev, rp2, ci2, v2)
    ones = torch.ones((n, 32), dtype=torch.float32, device=dev)
    plan2 = pkg.spmm.Plan(csr2, 32, sweep="force", sweep_panels_per_round=64)
    assert plan2.info.sweep_split_rows >= 1  # the long row is cut across panels and summed by the fix-up kernel
    Y = plan2.spmm(ones).cpu().numpy().astype(np.float64)
    sums = np.add.reduceat(np.concatenate([v2.astype(np.float64), [0.0]]), np.minimum(rp2[:-1], v2.size))
    sums[np.diff(rp2) == 0] = 0.0
    assert np.allclose(Y, sums[:, None], rtol=1e-5, atol=1e-6)


def test_sweep_plan_empty_matrix_and_empty_rows(pkg, dev):
    n = 130
    rp = np.zeros(n + 1, dtype=np.int32)
    csr = make_csr(pkg, dev, rp, np.zeros(0, dtype=np.int32), np.zeros(0, dtype=np.float32))
    d_X = torch.ones((n, 16), dtype=torch.float32, device=dev)
    plan = pkg.spmm.Plan(csr, 16, sweep="force", sweep_panels_per_round=4)
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    assert (Y == 0).all()


def test_sweep_plan_set_values_and_sources(pkg, orc, dev):
    rng = np.random.default_rng(9)
    n = 800
    for dt, K in (("f32", 16), ("f16", 64)):
        rp, ci, val, X = make_inputs(rng, n, 70, ((1, 700),), K, dt)
        csr = make_csr(pkg, dev, rp, ci, val)
        (d_X,) = to_dev(dev, X)
        plan = pkg.spmm.Plan(csr, K, sweep="force", sweep_panels_per_round=8)
        src = plan.array(pkg._cabi.MPS_PLAN_ARRAY_SW_SRC)
        real = src[src >= 0]
        assert np.array_equal(np.sort(real), np.arange(ci.size))  # every nonzero in exactly one slot
        stream = plan.array(pkg._cabi.MPS_PLAN_ARRAY_SW_STREAM).reshape(-1, 2)
        assert np.array_equal(stream[src >= 0, 1].view(np.float32), val[real].astype(np.float32))
        assert (stream[src < 0, 1] == 0).all()
        val2 = rng.random(ci.size).astype(val.dtype)
        (d_v2,) = to_dev(dev, val2)
        plan.set_values(d_v2)
        Y = plan.spmm(d_X)
        torch.cuda.synchronize()
        if dt == "f32":
            ref, scale = orc.spmm_f64(rp, ci, val2, X, want_abs=True)
            check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        else:
            ref, scale = orc.spmm_f64_f16in(rp, ci, val2, X, want_abs=True)
            check_fp16(Y.cpu().numpy(), ref, scale)
        nosrc = pkg.spmm.Plan(csr, K, sweep="force", sweep_panels_per_round=8, keep_sources=False)
        with pytest.raises(pkg._cabi.MpsError) as e:
            nosrc.set_values(d_v2)
        assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED


def test_sweep_plan_refuses_rows_that_start_between_dwords(pkg, dev):
    rng = np.random.default_rng(2)
    rp, ci, val, X = make_inputs(rng, 100, 5, (), 25, "f16")  # 50-byte rows
    csr = make_csr(pkg, dev, rp, ci, val)
    with pytest.raises(pkg._cabi.MpsError) as e:
        pkg.spmm.Plan(csr, 25, sweep="force")
    assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED


def test_sweep_plan_is_chosen_for_rows_that_leave_lanes_idle(pkg, orc, dev):
    # the library's own choice: one tile that the row does not fill, or whole 64 bytes; not rows of several tiles that
    # start anywhere in a line, not rows whose pitch is no multiple of 16 bytes
    rng = np.random.default_rng(12)
    n = 6000
    rp, ci = random_csr(rng, n, 30, p_empty=0.1, hub_rows=((3, 5000),))
    for dt, K, sweep in (("f32", 8, True), ("f32", 12, True), ("f32", 24, True), ("f32", 48, True), ("f32", 32, True),
                         ("f32", 41, False), ("f32", 36, False), ("f32", 100, False), ("f32", 18, False),
                         ("f16", 24, True), ("f16", 40, True), ("f16", 96, True), ("f16", 100, False), ("f16", 20, False)):
        npdt = np.float32 if dt == "f32" else np.float16
        val = rng.random(ci.size).astype(npdt)
        X = (rng.random((n, K)) * 2 - 1).astype(npdt)
        csr = make_csr(pkg, dev, rp, ci, val)
        (d_X,) = to_dev(dev, X)
        plan = pkg.spmm.Plan(csr, K)
        assert (plan.info.sweep_panels > 0) == sweep, (dt, K)
        Y = plan.spmm(d_X)
        torch.cuda.synchronize()
        if dt == "f32":
            ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
            check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        else:
            ref, scale = orc.spmm_f64_f16in(rp, ci, val, X, want_abs=True)
            check_fp16(Y.cpu().numpy(), ref, scale)


def test_sweep_plan_under_graph_capture(pkg, orc, dev):
    # a product launches kernels only: it can be captured, and every replay gives the eager bits
    rng = np.random.default_rng(4)
    rp, ci, val, X = make_inputs(rng, 3000, 40, ((9, 2800),), 32, "f32")
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, 32, sweep="force", sweep_panels_per_round=8)
    Y_eager = plan.spmm(d_X).clone()
    torch.cuda.synchronize()
    Y = torch.zeros_like(d_X)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        plan.spmm(d_X, out=Y)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.spmm(d_X, out=Y)
    for _ in range(3):
        Y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(Y, Y_eager)
