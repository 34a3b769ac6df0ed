"""Row-block plans on the GPU, through the C ABI: parity with the fp64 CPU loop
(the oracle), bit-identical repeats, value refresh, edge shapes."""
import numpy as np
import pytest
import torch

from tests.gpu_util import check_fp32, make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu

CASES = [
    # n, max_deg, hubs, steps, table_rows, block_rows, blocks_per_round
    (300, 40, ((5, 280), (150, 300)), 3, 16, 64, 4),
    (97, 12, (), 2, 8, 0, 2),
    (513, 60, ((0, 500), (512, 400)), 5, 32, 40, 8),
    (64, 64, ((10, 64),), 1, 64, 0, 1),
    (200, 5, (), 4, 4, 16, 256),
    (5000, 200, ((17, 4800), (4999, 3000)), 6, 256, 0, 64),
    (20000, 64, ((0, 15000),), 8, 0, 0, 0),
    # two rows far longer than a wavefront's run: every lane-group of several wavefronts ends in the same row
    (4096, 8, ((7, 4000), (2000, 3500)), 2, 512, 0, 1),
]


@pytest.mark.parametrize("case", CASES)
def test_rowblock_plan_matches_fp64_loop(pkg, orc, dev, case):
    n, max_deg, hubs, steps, table_rows, block_rows, per_round = case
    rng = np.random.default_rng(hash(case) % (2 ** 32))
    rp, ci = random_csr(rng, n, max_deg, p_empty=0.25, hub_rows=hubs)
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, 16, rowblock="force", rowblock_steps=steps, rowblock_table_rows=table_rows,
                         rowblock_block_rows=block_rows, rowblock_blocks_per_round=per_round)
    assert plan.info.rowblock_steps == steps
    Y = torch.full_like(d_X, float("nan"))
    plan.spmm(d_X, out=Y)
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    # repeats give the same bits, whatever Y held
    Y2 = torch.zeros_like(d_X)
    for _ in range(3):
        plan.spmm(d_X, out=Y2)
    torch.cuda.synchronize()
    assert torch.equal(Y, Y2)


def test_rowblock_plan_closed_forms(pkg, dev):
    # identity: Y = X; all-ones features: row sums
    n = 1000
    rp = np.arange(n + 1, dtype=np.int32)
    ci = np.arange(n, dtype=np.int32)
    val = np.ones(n, dtype=np.float32)
    rng = np.random.default_rng(1)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, 16, rowblock="force", rowblock_steps=3, rowblock_table_rows=100, rowblock_blocks_per_round=8)
    assert np.array_equal(plan.spmm(d_X).cpu().numpy(), X)
    rp2, ci2 = random_csr(rng, n, 50, hub_rows=((3, 900),))
    v2 = rng.random(ci2.size).astype(np.float32)
    csr2 = make_csr(pkg, dev, rp2, ci2, v2)
    ones = torch.ones((n, 16), dtype=torch.float32, device=dev)
    plan2 = pkg.spmm.Plan(csr2, 16, rowblock="force", rowblock_steps=4, rowblock_table_rows=64, rowblock_blocks_per_round=8)
    Y = plan2.spmm(ones).cpu().numpy().astype(np.float64)
    sums = np.add.reduceat(np.concatenate([v2.astype(np.float64), [0.0]]), np.minimum(rp2[:-1], v2.size))
    sums[np.diff(rp2) == 0] = 0.0
    assert np.allclose(Y, sums[:, None], rtol=1e-5, atol=1e-6)


def test_rowblock_plan_set_values_and_sources(pkg, orc, dev):
    rng = np.random.default_rng(9)
    n = 800
    rp, ci = random_csr(rng, n, 70, hub_rows=((1, 700),))
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, 16, rowblock="force", rowblock_steps=3, rowblock_table_rows=48, rowblock_blocks_per_round=8)
    val2 = rng.random(ci.size).astype(np.float32)
    (d_v2,) = to_dev(dev, val2)
    plan.set_values(d_v2)
    ref, scale = orc.spmm_f64(rp, ci, val2, X, want_abs=True)
    check_fp32(plan.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    lean = pkg.spmm.Plan(csr, 16, rowblock="force", rowblock_steps=3, rowblock_table_rows=48, rowblock_blocks_per_round=8,
                         keep_sources=False)
    assert lean.info.device_bytes < plan.info.device_bytes
    with pytest.raises(pkg._cabi.MpsError) as e:
        lean.set_values(d_v2)
    assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED
    # the device arrays are what the host-side builder makes
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, steps=3, table_rows=48, blocks_per_round=8)
    C = pkg._cabi
    for which, dt in ((C.MPS_PLAN_ARRAY_RB_BLOCK_ROW, np.int32), (C.MPS_PLAN_ARRAY_RB_META, np.int32),
                      (C.MPS_PLAN_ARRAY_RB_HOT_COLS, np.int32), (C.MPS_PLAN_ARRAY_RB_COLD_PACKED, np.uint32),
                      (C.MPS_PLAN_ARRAY_RB_COLD_BEGIN, np.int32), (C.MPS_PLAN_ARRAY_RB_HOT_SRC, np.int32)):
        assert np.array_equal(lean.array(which) if which != C.MPS_PLAN_ARRAY_RB_HOT_SRC else plan.array(which),
                              lay.array(which, dt))


@pytest.mark.parametrize("sparse", [False, True])
def test_rowblock_hot_stream_on_the_device_is_the_packed_form(pkg, orc, dev, sparse):
    """The device reads the hot stream in packed form (12 bytes per lane and round), with rows_advanced in two pieces
    (a lane-group's first window of a step lies up to a wavefront's run of rows from where the run starts; with mostly
    empty rows every window does): the product, new values, and the arrays the host builder makes."""
    rng = np.random.default_rng(77 + sparse)
    n = 3000
    if sparse:  # most rows empty
        rp, ci = random_csr(rng, n, 30, p_empty=0.97, hub_rows=((9, 2500), (2900, 2000)))
    else:
        rp, ci = random_csr(rng, n, 60, p_empty=0.05, hub_rows=((9, 2500),))
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    kw = dict(rowblock="force", rowblock_steps=2, rowblock_table_rows=64, rowblock_blocks_per_round=2)
    plan = pkg.spmm.Plan(csr, 16, **kw)
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, steps=2, table_rows=64, blocks_per_round=2)
    C = pkg._cabi
    hot = lay.array(C.MPS_PLAN_ARRAY_RB_HOT, np.uint32).reshape(-1, 2)
    assert (hot[:, 0] >> lay.info.hot_mark_shift).max() > 31  # the high piece of rows_advanced is in use
    assert plan.array(C.MPS_PLAN_ARRAY_RB_HOT).size == 0
    assert np.array_equal(plan.array(C.MPS_PLAN_ARRAY_RB_HOT_PACKED), lay.array(C.MPS_PLAN_ARRAY_RB_HOT_PACKED, np.uint32))
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    val2 = rng.random(ci.size).astype(np.float32)
    plan.set_values(to_dev(dev, val2)[0])
    ref2, scale2 = orc.spmm_f64(rp, ci, val2, X, want_abs=True)
    check_fp32(plan.spmm(d_X).cpu().numpy(), ref2, scale2, rel_elem=False)
    fresh = pkg.spmm.Plan(make_csr(pkg, dev, rp, ci, val2), 16, **kw)
    assert torch.equal(plan.spmm(d_X), fresh.spmm(d_X))
    assert np.array_equal(plan.array(C.MPS_PLAN_ARRAY_RB_HOT_PACKED), fresh.array(C.MPS_PLAN_ARRAY_RB_HOT_PACKED))
    # the cold stream likewise: packed on the device (ranges of 1,500 columns, windows at most 255 rows apart)
    assert plan.info.rowblock_cold_index_bits == 12 and plan.array(C.MPS_PLAN_ARRAY_RB_COLD).size == 0
    assert np.array_equal(plan.array(C.MPS_PLAN_ARRAY_RB_COLD_PACKED), fresh.array(C.MPS_PLAN_ARRAY_RB_COLD_PACKED))
    assert np.array_equal(fresh.array(C.MPS_PLAN_ARRAY_RB_COLD_PACKED), pkg.spmm.RowBlockLayout(rp, ci, val2, steps=2, table_rows=64, blocks_per_round=2).array(C.MPS_PLAN_ARRAY_RB_COLD_PACKED, np.uint32))


def test_rowblock_cold_stream_stays_unpacked_when_it_does_not_fit(pkg, orc, dev):
    """Ranges wider than 32,768 columns (one step over 40,000 columns) or windows further apart than the pieces hold
    leave the cold stream as 8-byte entries: the other instantiation of the kernel reads them."""
    rng = np.random.default_rng(5)
    n = 40000
    rp, ci = random_csr(rng, n, 6, p_empty=0.3, hub_rows=((3, 30000),))
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    C = pkg._cabi
    plan = pkg.spmm.Plan(csr, 16, rowblock="force", rowblock_steps=1, rowblock_table_rows=64, rowblock_blocks_per_round=8)
    assert plan.info.rowblock_cold_index_bits == 0 and plan.array(C.MPS_PLAN_ARRAY_RB_COLD_PACKED).size == 0
    lay = pkg.spmm.RowBlockLayout(rp, ci, val, steps=1, table_rows=64, blocks_per_round=8)
    assert np.array_equal(plan.array(C.MPS_PLAN_ARRAY_RB_COLD), lay.array(C.MPS_PLAN_ARRAY_RB_COLD, np.uint32))
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(plan.spmm(d_X, out=torch.full_like(d_X, float("nan"))).cpu().numpy(), ref, scale, rel_elem=False)
    val2 = rng.random(ci.size).astype(np.float32)
    plan.set_values(to_dev(dev, val2)[0])
    ref2, scale2 = orc.spmm_f64(rp, ci, val2, X, want_abs=True)
    check_fp32(plan.spmm(d_X).cpu().numpy(), ref2, scale2, rel_elem=False)
    # mostly empty rows, 15-bit ranges (one 4-bit piece... a window 20 rows from the last one does not fit 4 bits)
    rp3, ci3 = random_csr(rng, 30000, 40, p_empty=0.99, hub_rows=((9, 25000), (29000, 20000)))
    val3 = rng.random(ci3.size).astype(np.float32)
    X3 = (rng.random((30000, 16)) * 2 - 1).astype(np.float32)
    plan3 = pkg.spmm.Plan(make_csr(pkg, dev, rp3, ci3, val3), 16, rowblock="force", rowblock_steps=1, rowblock_table_rows=64,
                          rowblock_blocks_per_round=2)
    assert plan3.info.rowblock_cold_index_bits == 0
    ref3, scale3 = orc.spmm_f64(rp3, ci3, val3, X3, want_abs=True)
    check_fp32(plan3.spmm(to_dev(dev, X3)[0]).cpu().numpy(), ref3, scale3, rel_elem=False)


def test_rowblock_plan_rejects_other_shapes(pkg, dev):
    rng = np.random.default_rng(2)
    rp, ci = random_csr(rng, 100, 10)
    val = rng.random(ci.size).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    with pytest.raises(pkg._cabi.MpsError) as e:
        pkg.spmm.Plan(csr, 32, rowblock="force")
    assert e.value.status == pkg._cabi.MPS_ERR_UNSUPPORTED
    bad = make_csr(pkg, dev, rp, np.where(np.arange(ci.size) == 3, 100, ci).astype(np.int32), val)
    with pytest.raises(pkg._cabi.MpsError) as e:
        pkg.spmm.Plan(bad, 16, rowblock="force")
    assert e.value.status == pkg._cabi.MPS_ERR_INVALID_CSR


def test_rowblock_plan_power_law_graph(pkg, orc, dev):
    # the benchmark graph's shape at a tenth of its size; the library picks the plan kind and its parameters
    rp, ci, _ = pkg.graphs.generate("chunglu:n=60000,nnz=12000000,gamma=2.1,dmax=8000", seed=3)
    n, nnz = rp.size - 1, ci.size
    val = pkg.graphs.fill_uniform_f32(nnz, 11, 0.0, 1.0)
    X = pkg.graphs.fill_uniform_f32(n * 16, 13, -1.0, 1.0).reshape(n, 16)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, 16, rowblock="force")
    assert plan.info.rowblock_blocks > 0 and plan.info.hot_nnz > 0
    Y = plan.spmm(d_X)
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    Y2 = plan.spmm(d_X)
    assert torch.equal(Y, Y2)


def test_uniform_matrix_gets_a_rowblock_plan_too(pkg, orc, dev):
    # columns used evenly: the LDS tables serve a twentieth of the nonzeros, but a block still has 20,000
    # nonzeros per step and the gathers of a step stay in L2, so the library builds the row-block plan
    rp, ci, _ = pkg.graphs.generate("er:n=200000,deg=130", seed=5)
    n, nnz = rp.size - 1, ci.size
    val = pkg.graphs.fill_uniform_f32(nnz, 11, 0.0, 1.0)
    X = pkg.graphs.fill_uniform_f32(n * 16, 13, -1.0, 1.0).reshape(n, 16)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, 16)
    i = plan.info
    assert i.rowblock_steps == 5 and i.hot_nnz < 0.25 * nnz  # 12.8 MB of X at 3 MiB a step
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(plan.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    slabs = pkg.spmm.Plan(csr, 16, rowblock="off")
    assert slabs.info.rowblock_steps == 0 and slabs.info.num_slabs > 1
    check_fp32(slabs.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)


@pytest.mark.parametrize("kind", ["short_rows", "banded", "long_row"])
def test_matrices_that_stay_with_the_slab_plans(pkg, orc, dev, kind):
    """No row-block plan unless asked for: many short rows without busy columns (a million rows of 8,
    columns used evenly), columns that stay near the diagonal but not near enough for tables of a
    block's own (a band of 12,000 columns either side: 8 tables would serve half of it, and with global
    tables every block would idle through the steps of the other column ranges), and a row that is
    many times a CU's share of the nonzeros (rows are not cut across blocks)."""
    rng = np.random.default_rng(3)
    if kind == "short_rows":
        rp, ci, _ = pkg.graphs.generate("er:n=1000000,deg=8", seed=5)
    elif kind == "long_row":
        rp, ci, _ = pkg.graphs.generate("chunglu:n=262144,nnz=1000000,gamma=2.1,dmax=50000", seed=5)
        assert np.diff(rp).max() > 2 * ci.size / 256
    else:
        rp, ci, _ = pkg.graphs.generate("band:n=120000,deg=48,width=12000", seed=5)
    n, nnz = rp.size - 1, ci.size
    val = pkg.graphs.fill_uniform_f32(nnz, 11, 0.0, 1.0)
    X = pkg.graphs.fill_uniform_f32(n * 16, 13, -1.0, 1.0).reshape(n, 16)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, 16)
    assert plan.info.rowblock_steps == 0
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(plan.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    forced = pkg.spmm.Plan(csr, 16, rowblock="force")
    assert forced.info.rowblock_steps > 0
    check_fp32(forced.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)


@pytest.mark.parametrize("forced", [True, False])
def test_local_tables_on_a_block_diagonal_matrix(pkg, orc, dev, forced):
    """Columns that stay near the diagonal: every block gets a table of consecutive columns of its own (one step,
    the table read straight from X) - asked for with MPS_PLAN_LOCAL_TABLES, or chosen by the library where such
    tables serve most of the nonzeros."""
    rp, ci, _ = pkg.graphs.generate("blockdiag:blocks=300,min=100,max=600,deg=5", seed=9)
    n, nnz = rp.size - 1, ci.size
    val = pkg.graphs.fill_uniform_f32(nnz, 11, 0.0, 1.0)
    X = pkg.graphs.fill_uniform_f32(n * 16, 13, -1.0, 1.0).reshape(n, 16)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    kw = dict(rowblock="force", local_tables=True, rowblock_steps=1, rowblock_table_rows=256, rowblock_block_rows=300) if forced else {}
    plan = pkg.spmm.Plan(csr, 16, **kw)
    i = plan.info
    assert i.rowblock_local_tables == 1 and i.rowblock_steps == 1
    assert (i.hot_nnz > 0.9 * nnz) == (not forced)  # one table of 256 rows misses many of a block's columns
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=True)
    assert torch.equal(Y, plan.spmm(d_X))
    base = plan.array(pkg._cabi.MPS_PLAN_ARRAY_RB_TABLE_BASE)
    assert base.size == i.rowblock_blocks and (base >= 0).all() and (base + i.rowblock_steps * i.rowblock_table_rows <= n).all()
    # new values through the source indices
    val2 = pkg.graphs.fill_uniform_f32(nnz, 21, 0.0, 1.0)
    plan.set_values(torch.from_numpy(val2).to(dev))
    ref2, scale2 = orc.spmm_f64(rp, ci, val2, X, want_abs=True)
    check_fp32(plan.spmm(d_X).cpu().numpy(), ref2, scale2, rel_elem=True)


def test_local_tables_of_several_steps_on_a_banded_matrix(pkg, orc, dev):
    """A band of 2,000 columns either side of the diagonal: the library gives every block three tables of
    consecutive columns, one per step, and nearly every nonzero is gathered from LDS."""
    rp, ci, _ = pkg.graphs.generate("band:n=120000,deg=48,width=2000", seed=5)
    n = rp.size - 1
    nnz = ci.size
    val = pkg.graphs.fill_uniform_f32(nnz, 11, 0.0, 1.0)
    X = pkg.graphs.fill_uniform_f32(n * 16, 13, -1.0, 1.0).reshape(n, 16)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, 16)
    i = plan.info
    assert i.rowblock_local_tables == 1 and i.rowblock_steps == 3 and i.hot_nnz > 0.95 * nnz
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    assert torch.equal(Y, plan.spmm(d_X))
    slabs = pkg.spmm.Plan(csr, 16, rowblock="off")
    check_fp32(slabs.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)


def test_rowblock_small_plan_does_not_lower_the_lds_limit_of_a_large_one(pkg, orc, dev):
    # The dynamic-LDS limit belongs to the kernel, not to a plan: a plan with a full table, then one with a
    # 16-row table, then the first again - same bits as before the second one existed.
    rng = np.random.default_rng(77)
    n = 6000
    rp, ci = random_csr(rng, n, 90, hub_rows=((11, 5500),))
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 16)) * 2 - 1).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    big = pkg.spmm.Plan(csr, 16, rowblock="force", rowblock_steps=2, rowblock_blocks_per_round=8)
    assert big.info.rowblock_table_rows > 1000  # what fits beside the accumulators: well over 64 KiB of LDS
    Y0 = big.spmm(d_X).clone()
    torch.cuda.synchronize()
    small = pkg.spmm.Plan(csr, 16, rowblock="force", rowblock_steps=2, rowblock_table_rows=16, rowblock_blocks_per_round=8)
    Ys = small.spmm(d_X)
    torch.cuda.synchronize()
    Y1 = big.spmm(d_X, out=torch.full_like(d_X, float("nan")))  # raises if the launch is refused
    torch.cuda.synchronize()
    assert torch.equal(Y0, Y1)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y1.cpu().numpy(), ref, scale, rel_elem=False)
    check_fp32(Ys.cpu().numpy(), ref, scale, rel_elem=False)
