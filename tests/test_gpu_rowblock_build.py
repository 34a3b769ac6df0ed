"""Row-block plans built with the passes over the nonzeros on the device against the same plans built on the host
(MPS_PLAN_HOST_BUILD): every array of the layout, the plan's description and the product must be the same bits."""
import numpy as np
import pytest
import torch

from tests.gpu_util import check_fp32, make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu

CASES = [
    # n, max_deg, hubs, p_empty, steps, table_rows, block_rows, blocks_per_round
    (300, 40, ((5, 280), (150, 300)), 0.25, 3, 16, 64, 4),
    (97, 12, (), 0.25, 2, 8, 0, 2),
    (513, 60, ((0, 500), (512, 400)), 0.25, 5, 32, 40, 8),
    (64, 64, ((10, 64),), 0.0, 1, 64, 0, 1),
    (200, 5, (), 0.5, 4, 4, 16, 256),                       # more blocks than rows with nonzeros can fill
    (5000, 200, ((17, 4800), (4999, 3000)), 0.25, 6, 256, 0, 64),
    (20000, 64, ((0, 15000),), 0.1, 8, 0, 0, 0),            # the library's table size and blocks
    (4096, 8, ((7, 4000), (2000, 3500)), 0.25, 2, 512, 0, 1),
    (3000, 30, ((9, 2500), (2900, 2000)), 0.97, 2, 64, 0, 2),  # mostly empty rows: windows far apart
    (30000, 90, ((100, 20000),), 0.0, 0, 0, 0, 0),          # everything chosen by the library
    (2000, 50, (), 0.2, 64, 8, 0, 4),                       # as many steps as the device passes take
    (5, 3, (), 0.0, 1, 4, 0, 1),
]

ARRAYS = ["RB_BLOCK_ROW", "RB_HOT_COLS", "RB_META", "RB_WAVE_BASE", "RB_HOT_SRC", "RB_COLD_SRC", "RB_HOT_PACKED",
          "RB_COLD_PACKED", "RB_COLD", "RB_COLD_BEGIN", "RB_TABLE_BASE"]


def both_plans(pkg, dev, rp, ci, val, **kw):
    csr = make_csr(pkg, dev, rp, ci, val)
    return csr, pkg.spmm.Plan(csr, 16, rowblock="force", **kw), pkg.spmm.Plan(csr, 16, rowblock="force", host_build=True, **kw)


def same_plan(pkg, a, b):
    ia, ib = a.info, b.info
    assert ib.built_on_device == 0
    for name, _ in ia._fields_:
        assert name == "built_on_device" or getattr(ia, name) == getattr(ib, name), name
    for name in ARRAYS:
        which = getattr(pkg._cabi, "MPS_PLAN_ARRAY_" + name)
        assert np.array_equal(a.array(which), b.array(which)), name


@pytest.mark.parametrize("case", CASES)
def test_device_passes_build_the_host_builders_plan(pkg, orc, dev, case):
    n, max_deg, hubs, p_empty, steps, table_rows, block_rows, per_round = case
    rng = np.random.default_rng(abs(hash(case)) % (2 ** 32))
    rp, ci = random_csr(rng, n, max_deg, p_empty=p_empty, hub_rows=hubs)
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    csr, plan, host = both_plans(pkg, dev, rp, ci, val, rowblock_steps=steps, rowblock_table_rows=table_rows,
                                 rowblock_block_rows=block_rows, rowblock_blocks_per_round=per_round)
    assert plan.info.rowblock_steps > 0
    same_plan(pkg, plan, host)
    (d_X,) = to_dev(dev, X)
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    assert torch.equal(Y, host.spmm(d_X))
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    # new values reach the same slots
    val2 = rng.random(ci.size).astype(np.float32)
    (d_v2,) = to_dev(dev, val2)
    plan.set_values(d_v2)
    host.set_values(d_v2)
    same_plan(pkg, plan, host)


def test_plans_that_the_host_passes_build(pkg, orc, dev):
    """Local tables, more steps than the device passes rank, a cold stream that cannot be packed: the host builder
    takes over, and says nothing of it."""
    rng = np.random.default_rng(31)
    n = 6000
    rp, ci = random_csr(rng, n, 40, p_empty=0.1)
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    (d_X,) = to_dev(dev, X)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    for kw in (dict(local_tables=True, rowblock_steps=2, rowblock_table_rows=64),
               dict(rowblock_steps=100, rowblock_table_rows=8, rowblock_blocks_per_round=8)):
        csr, plan, host = both_plans(pkg, dev, rp, ci, val, **kw)
        same_plan(pkg, plan, host)
        check_fp32(plan.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    n2 = 40000  # one step over 40,000 columns: ranges wider than a packed entry holds
    rp2, ci2 = random_csr(rng, n2, 6, p_empty=0.3, hub_rows=((3, 30000),))
    val2 = rng.random(ci2.size).astype(np.float32)
    csr, plan, host = both_plans(pkg, dev, rp2, ci2, val2, rowblock_steps=1, rowblock_table_rows=64, rowblock_blocks_per_round=8)
    assert plan.info.rowblock_cold_index_bits == 0
    same_plan(pkg, plan, host)
    # windows further apart than the pieces of a packed entry hold: found while placing, then built again on the host
    rp3, ci3 = random_csr(rng, 30000, 40, p_empty=0.99, hub_rows=((9, 25000), (29000, 20000)))
    val3 = rng.random(ci3.size).astype(np.float32)
    csr, plan, host = both_plans(pkg, dev, rp3, ci3, val3, rowblock_steps=1, rowblock_table_rows=64, rowblock_blocks_per_round=2)
    assert plan.info.rowblock_cold_index_bits == 0
    same_plan(pkg, plan, host)


def test_device_passes_on_random_shapes(pkg, dev):
    """Forty matrices and parameter sets drawn at random (sizes, row lengths, empty rows, long rows, steps, table and
    block sizes): the device passes and the host passes agree on every one, or turn it away with the same status."""
    rng = np.random.default_rng(2024)
    built = 0
    for trial in range(40):
        n = int(rng.choice([7, 60, 333, 1500, 6000, 25000]))
        max_deg = int(rng.choice([1, 3, 9, 40, 150]))
        hubs = tuple((int(rng.integers(0, n)), int(rng.integers(1, n + 1))) for _ in range(int(rng.integers(0, 3))))
        hubs = tuple(dict(hubs).items())  # (one entry per row)
        rp, ci = random_csr(rng, n, max_deg, p_empty=float(rng.choice([0.0, 0.3, 0.9])), hub_rows=hubs)
        val = rng.random(ci.size).astype(np.float32)
        kw = dict(rowblock_steps=int(rng.choice([0, 1, 2, 5, 17, 40])), rowblock_table_rows=int(rng.choice([0, 4, 24, 200, 1024])),
                  rowblock_block_rows=int(rng.choice([0, 0, 8, 100])), rowblock_blocks_per_round=int(rng.choice([0, 1, 3, 16, 256])))
        csr = make_csr(pkg, dev, rp, ci, val)
        status = []
        plans = []
        for host in (False, True):
            try:
                plans.append(pkg.spmm.Plan(csr, 16, rowblock="force", host_build=host, **kw))
                status.append(0)
            except pkg._cabi.MpsError as e:
                status.append(e.status)
        assert status[0] == status[1], (trial, n, max_deg, hubs, kw, status)
        if status[0] == 0:
            same_plan(pkg, plans[0], plans[1])
            X = torch.rand((n, 16), dtype=torch.float32, device=dev)
            assert torch.equal(plans[0].spmm(X), plans[1].spmm(X)), (trial, n, kw)
            built += 1
    assert built >= 25
