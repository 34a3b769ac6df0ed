"""The five benchmark workloads at full size on the GPU: against the oracle's fp64 row
loop (OpenMP, seconds on the host) and through size-independent properties
(all-ones features give row sums; linearity; plan and CSR entry points agree)."""
import numpy as np
import pytest
import torch

from gpu_util import check_fp32, make_csr, to_dev

pytestmark = pytest.mark.gpu


def workload(pkg, spec, K, half=False):
    g = pkg.graphs
    rp, ci, _ = g.generate(spec, seed=1)
    n = rp.size - 1
    fill = g.fill_uniform_f16 if half else g.fill_uniform_f32
    return rp, ci, fill(ci.size, 11, 0.0, 1.0), fill(n * K, 13, -1.0, 1.0).reshape(n, K)


def row_sums(rp, val):
    s = np.add.reduceat(np.concatenate([val.astype(np.float64), [0.0]]), rp[:-1])
    s[np.diff(rp) == 0] = 0.0
    return s


def test_power_law_config_full_size(pkg, orc, dev):
    # config 2: Chung-Lu, N = 232,965, nnz ~ 114.6 M, fp32, K = 16
    K = 16
    rp, ci, val, X = workload(pkg, pkg.graphs.CONFIG_SPECS["chunglu_233k"], K)
    assert rp.size - 1 == 232965 and abs(ci.size - 114.6e6) < 0.5e6
    csr = make_csr(pkg, dev, rp, ci, val)
    csr.validate()
    (d_X,) = to_dev(dev, X)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    plan = pkg.spmm.Plan(csr, K)
    # the library's own choice here: a row-block plan (rows summed in LDS, more than half of the nonzeros
    # gathered from LDS tables), one block per CU
    assert plan.info.rowblock_steps > 0 and plan.info.rowblock_blocks % 256 == 0 and plan.info.hot_nnz > 0.5 * ci.size
    Yp = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    # without row blocks: 5 slabs of 3 MiB, 1,728 hot columns per slab (over a third of the nonzeros)
    slab_plan = pkg.spmm.Plan(csr, K, rowblock="off")
    assert slab_plan.info.num_slabs == 5 and slab_plan.info.hot_rows == 1728 and slab_plan.info.hot_nnz > 0.3 * ci.size
    Ys = slab_plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    slab_plan.close()
    sched = pkg.spmm.generate_mp_sched(csr.row_ptr, csr.nnz)
    # the partition of the caller's CSR is the reference split, bit for bit, at this size too
    xs, ys = orc.partition_coords(rp, ci.size, sched.P)
    assert np.array_equal(sched.coord_x.cpu().numpy(), xs) and np.array_equal(sched.coord_y.cpu().numpy(), ys)
    Yc = pkg.spmm.spmm_merge_path(csr, d_X, sched, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    for Y in (Yp, Ys, Yc):
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    assert torch.equal(Yp, plan.spmm(d_X))  # same bits on a second launch
    # all-ones features: every column of Y is the row sum of the values
    ones = torch.ones_like(d_X)
    Y1 = plan.spmm(ones).cpu().numpy()
    rs = row_sums(rp, val)
    assert np.abs(Y1 - rs[:, None]).max() <= 1e-5 * rs.max()
    assert (Y1 == Y1[:, :1]).all()
    # linearity: A (2 X - 3 X2) = 2 A X - 3 A X2
    X2 = torch.from_numpy(pkg.graphs.fill_uniform_f32(X.size, 17, -1.0, 1.0).reshape(X.shape)).to(dev)
    lhs = plan.spmm(2 * d_X - 3 * X2)
    rhs = 2 * Yp - 3 * plan.spmm(X2)
    bound = torch.from_numpy((2e-5 * 5 * scale + 1e-5).astype(np.float32)).to(dev)
    assert ((lhs - rhs).abs() <= bound).all()


@pytest.mark.parametrize("spec,big_slabs", [("chunglu:n=1000000,nnz=60000000,gamma=2.1,dmax=30000", True),
                                            ("er:n=1000000,deg=60", False)])
def test_slab_size_follows_the_skew_of_the_matrix(pkg, orc, dev, spec, big_slabs):
    """X of 64 MB: a power-law matrix gets slabs far beyond the L2 (its popular columns stay
    cached), a uniform one slabs of at most 6 MiB; both plans give the right product."""
    K = 16
    rp, ci, val, X = workload(pkg, spec, K)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, K)
    i = plan.info
    slab_bytes = i.slab_cols * K * 4
    assert i.num_slabs > 1 and i.hot_rows == 0
    assert (slab_bytes > (8 << 20)) == big_slabs and (big_slabs or slab_bytes <= (6 << 20) + 4096)
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    plan.close()


@pytest.mark.parametrize("K", [16, 256])
def test_rmat_config_full_size(pkg, orc, dev, K):
    # config 4: R-MAT scale 20, edge factor 16, deduplicated; ends of the K sweep
    rp, ci, val, X = workload(pkg, pkg.graphs.CONFIG_SPECS["rmat_s20"], K)
    assert rp.size - 1 == 1 << 20
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    plan = pkg.spmm.Plan(csr, K)
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    sched = pkg.spmm.generate_mp_sched(csr.row_ptr, csr.nnz)
    Yc = pkg.spmm.spmm_merge_path(csr, d_X, sched, out=torch.full_like(d_X, float("nan")))
    check_fp32(Yc.cpu().numpy(), ref, scale, rel_elem=False)


def test_block_diagonal_config_full_size(pkg, orc, dev):
    # config 3: 1,178 disjoint random-geometric blocks, fp32, K = 16; rows are short, so the
    # per-element bar (1e-5 relative, 1e-6 absolute) applies literally
    K = 16
    rp, ci, val, X = workload(pkg, pkg.graphs.CONFIG_SPECS["blockdiag_1178"], K)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    for Y in (pkg.spmm.Plan(csr, K).spmm(d_X),
              pkg.spmm.spmm_merge_path(csr, d_X, pkg.spmm.generate_mp_sched(csr.row_ptr, csr.nnz))):
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=True)
    # block structure: a row only sees columns of its own block, so zeroing X outside a block
    # leaves that block's rows unchanged
    cut = 50000
    lo = int(ci[rp[0]:rp[cut]].max()) + 1
    Xz = d_X.clone()
    Xz[lo:] = 0
    Yz = pkg.spmm.Plan(csr, K).spmm(Xz)
    Y0 = pkg.spmm.Plan(csr, K).spmm(d_X)
    assert torch.equal(Yz[:cut], Y0[:cut])


def test_fp16_config_full_size(pkg, orc, dev):
    # config 5: R-MAT scale 22, half values and features, K = 64, fp32 accumulation
    K = 64
    rp, ci, val, X = workload(pkg, pkg.graphs.CONFIG_SPECS["rmat_s22"], K, half=True)
    assert rp.size - 1 == 1 << 22
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    ref, scale = orc.spmm_f64_f16in(rp, ci, val, X, want_abs=True)
    plan = pkg.spmm.Plan(csr, K)
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    Yh = Y.cpu().numpy().astype(np.float64)
    err = np.abs(Yh - ref)
    assert np.isfinite(Yh).all()
    assert (err <= 2e-2 * np.abs(ref) + 2e-5 * scale + 1e-6).all()      # the stated bar
    assert (err <= 2.0 ** -10 * np.abs(ref) + 1e-5 * scale + 1e-7).all()  # one half rounding
    sched = pkg.spmm.generate_mp_sched(csr.row_ptr, csr.nnz)
    Yc = pkg.spmm.spmm_merge_path(csr, d_X, sched).cpu().numpy().astype(np.float64)
    assert (np.abs(Yc - ref) <= 2.0 ** -10 * np.abs(ref) + 1e-5 * scale + 1e-7).all()
