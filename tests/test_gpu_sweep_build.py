"""Sweep plans built with the passes over the nonzeros on the device against the same plans built on the host
(MPS_PLAN_HOST_BUILD): every array of the layout, the plan's description and the product must be the same bits."""
import numpy as np
import pytest
import torch

from tests.gpu_util import make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu

CASES = [
    # n, max_deg, hubs, p_empty, K, dtype, piece, acc_rows, panels_per_round, together
    (300, 40, ((5, 280), (150, 300)), 0.25, 16, "f32", 0, 0, 4, 0),
    (97, 12, (), 0.25, 32, "f32", 4, 0, 2, 0),
    (513, 60, ((0, 500), (512, 400)), 0.25, 64, "f32", 8, 64, 8, 0),     # several rounds of panels, two tiles
    (200, 5, (), 0.5, 16, "f32", 2, 16, 256, 0),                          # more panels than rows
    (5000, 200, ((17, 4800), (4999, 3000)), 0.25, 128, "f32", 0, 0, 64, 0),  # rows cut across panels
    (20000, 64, ((0, 15000),), 0.1, 16, "f32", 0, 0, 0, 0),
    (4096, 8, ((7, 4000), (2000, 3500)), 0.25, 256, "f32", 0, 0, 16, 0),
    (3000, 30, ((11, 2500),), 0.25, 64, "f16", 0, 0, 8, 0),
    (1000, 20, (), 0.25, 32, "f16", 0, 0, 4, 0),
    (3000, 40, ((5, 2800),), 0.25, 16, "f32", 0, 0, 8, 1),
    (3000, 40, ((5, 2800),), 0.25, 32, "f32", 0, 0, 8, 2),
    (60000, 30, ((9, 50000),), 0.3, 16, "f32", 0, 0, 32, 0),
    (1, 1, (), 0.0, 16, "f32", 0, 0, 1, 0),
    (130, 0, (), 1.0, 16, "f32", 0, 0, 4, 0),                             # no nonzeros at all
]

ARRAYS = ["SW_PANEL_PTR", "SW_ROWS", "SW_PIECE_PTR", "SW_WAVE_META", "SW_PANEL_ROUNDS", "SW_STREAM", "SW_SRC",
          "SW_SPLIT_ROW", "SW_SPLIT_PTR"]


def same_plan(pkg, a, b):
    ia, ib = a.info, b.info
    assert ib.built_on_device == 0
    for name, _ in ia._fields_:
        assert name == "built_on_device" or getattr(ia, name) == getattr(ib, name), name
    for name in ARRAYS:
        which = getattr(pkg._cabi, "MPS_PLAN_ARRAY_" + name)
        assert np.array_equal(a.array(which), b.array(which)), name


@pytest.mark.parametrize("case", CASES)
def test_device_passes_build_the_host_builders_sweep_plan(pkg, dev, case):
    n, max_deg, hubs, p_empty, K, dt, piece, acc_rows, per_round, together = case
    rng = np.random.default_rng(abs(hash(case)) % (2 ** 32))
    if max_deg == 0:
        rp, ci = np.zeros(n + 1, dtype=np.int32), np.zeros(0, dtype=np.int32)
    else:
        rp, ci = random_csr(rng, n, max_deg, p_empty=p_empty, hub_rows=hubs)
    npdt = np.float32 if dt == "f32" else np.float16
    val = rng.random(ci.size).astype(npdt)
    X = (rng.random((n, K)) * 2 - 1).astype(npdt)
    csr = make_csr(pkg, dev, rp, ci, val)
    kw = dict(sweep="force", sweep_piece=piece, sweep_acc_rows=acc_rows, sweep_panels_per_round=per_round, sweep_together=together)
    plan = pkg.spmm.Plan(csr, K, **kw)
    host = pkg.spmm.Plan(csr, K, host_build=True, **kw)
    assert plan.info.sweep_panels > 0
    same_plan(pkg, plan, host)
    (d_X,) = to_dev(dev, X)
    assert torch.equal(plan.spmm(d_X), host.spmm(d_X))
    if ci.size:
        val2 = rng.random(ci.size).astype(npdt)
        (d_v2,) = to_dev(dev, val2)
        plan.set_values(d_v2)
        host.set_values(d_v2)
        same_plan(pkg, plan, host)


def test_device_passes_on_random_shapes(pkg, dev):
    """Thirty matrices and parameter sets drawn at random: the device passes and the host passes agree on every one,
    or turn it away with the same status."""
    rng = np.random.default_rng(77)
    built = 0
    for trial in range(30):
        n = int(rng.choice([5, 70, 400, 2500, 9000, 40000]))
        max_deg = int(rng.choice([1, 4, 12, 60, 200]))
        hubs = dict((int(rng.integers(0, n)), int(rng.integers(1, n + 1))) for _ in range(int(rng.integers(0, 3))))
        rp, ci = random_csr(rng, n, max_deg, p_empty=float(rng.choice([0.0, 0.3, 0.9])), hub_rows=tuple(hubs.items()))
        K, dt = [(16, "f32"), (32, "f32"), (64, "f32"), (192, "f32"), (32, "f16"), (64, "f16"), (128, "f16")][int(rng.integers(0, 7))]
        npdt = np.float32 if dt == "f32" else np.float16
        val = rng.random(ci.size).astype(npdt)
        kw = dict(sweep="force", sweep_piece=int(rng.choice([0, 0, 3, 20])), sweep_acc_rows=int(rng.choice([0, 0, 24, 200])),
                  sweep_panels_per_round=int(rng.choice([0, 1, 5, 64, 256])), sweep_together=int(rng.choice([0, 1, 2])))
        csr = make_csr(pkg, dev, rp, ci, val)
        status, plans = [], []
        for host in (False, True):
            try:
                plans.append(pkg.spmm.Plan(csr, K, host_build=host, **kw))
                status.append(0)
            except pkg._cabi.MpsError as e:
                status.append(e.status)
        assert status[0] == status[1], (trial, n, max_deg, hubs, K, dt, kw, status)
        if status[0] == 0:
            same_plan(pkg, plans[0], plans[1])
            X = torch.rand((n, K), device=dev).to(torch.float32 if dt == "f32" else torch.float16)
            assert torch.equal(plans[0].spmm(X), plans[1].spmm(X)), (trial, n, K, kw)
            built += 1
    assert built >= 20
