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


def outside_literal_bar(Y, ref):
    """elements that miss |err| <= 1e-5 |ref| + 1e-6, the bar as the benchmark states it"""
    return np.abs(Y.astype(np.float64) - ref) > 1e-5 * np.abs(ref) + 1e-6


def cpu_fp32_loops(orc, rp, ci, val, X, P):
    """The plain sequential fp32 loops on the CPU: the row loop (test/compare.h:18-31 run in fp32) and the
    merge-path order (src/MergePathSpMM.cu:426-477, one thread after the other)."""
    return orc.spmm_f32_mt(rp, ci, val, X), orc.spmm_mergepath_f32(rp, ci, val, X, P)


def check_against_cpu_fp32_loops(loops, ref, Yg):
    """Where the GPU result misses the literal per-element bar (rows whose terms cancel), it does so no more
    often and by no more than the plain sequential fp32 loops on the CPU do.  Row by row either side can be
    the lucky one (the rounding errors of two summation orders are nearly independent), so the comparison
    by rows allows a handful of exceptions (two rows in a hundred beyond twice the CPU loops' error, none beyond
    four times: the row-block plan on R-MAT has 2 of 471 at up to 2.4 times, with a third of the row loop's
    misses in total; the sweep plan 10 of 770, with half of the row loop's misses - the rows are picked by the
    GPU's misses, which favours the CPU loops on them) and the totals allow none.  Returns the three counts."""
    Yrow, Ymp = loops
    miss_g = outside_literal_bar(Yg, ref)
    counts = [int(miss_g.sum()), int(outside_literal_bar(Yrow, ref).sum()), int(outside_literal_bar(Ymp, ref).sum())]
    # fewer misses than the row loop, the order the reference checks itself against (test/compare.h:18-31).
    # The merge-path loop cuts long rows into P-dependent pieces, a blocked summation of its own: it can
    # miss on fewer elements than the GPU (R-MAT, K = 64: 1,223 against 3,308) or on more, so for it
    # the sizes of the errors are compared below, not the counts.
    assert counts[0] <= counts[1], counts
    # on the rows that hold a GPU miss: the GPU's largest error in the row against the CPU loops' largest
    rows = np.nonzero(miss_g.any(axis=1))[0]
    if rows.size:
        eg = np.abs(Yg[rows].astype(np.float64) - ref[rows]).max(axis=1)
        er = np.abs(Yrow[rows].astype(np.float64) - ref[rows]).max(axis=1)
        em = np.abs(Ymp[rows].astype(np.float64) - ref[rows]).max(axis=1)
        within = eg <= 2.0 * np.maximum(er, em)
        print("outside the literal bar: GPU %d, row loop %d, merge-path loop %d elements" % tuple(counts))
        print("rows with a GPU miss: %d; within 2x of the CPU loops: %d; worst ratio %.2f; largest error GPU %.3e, "
              "row loop %.3e, merge-path loop %.3e; mean error GPU %.3e, row loop %.3e, merge-path loop %.3e"
              % (rows.size, int(within.sum()), float((eg / np.maximum(np.maximum(er, em), 1e-30)).max()),
                 eg.max(), er.max(), em.max(), eg.mean(), er.mean(), em.mean()))
        assert within.sum() >= 0.98 * rows.size and (eg <= 4.0 * np.maximum(er, em)).all()
        assert eg.max() <= 2.0 * max(er.max(), em.max()) and eg.mean() <= 2.0 * min(er.mean(), em.mean())
    return counts


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
    # both entry streams in packed form (a step's cold columns span fewer than 16,384 ids): without the source
    # indices that this plan keeps for mps_plan_set_values, it is smaller than the CSR arrays
    sources = 4 * (plan.info.rowblock_hot_slots + plan.info.rowblock_cold_slots)
    assert plan.info.rowblock_cold_index_bits == 14 and plan.info.device_bytes - sources < 8 * ci.size + 4 * rp.size
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
    loops = cpu_fp32_loops(orc, rp, ci, val, X, sched.P)
    for Y in (Yp, Ys, Yc):
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        # rows of ~500 terms of both signs: some elements miss the literal bar in any fp32 summation order;
        # the GPU misses it on fewer elements, and by less, than the CPU's sequential fp32 loops
        check_against_cpu_fp32_loops(loops, ref, Y.cpu().numpy())
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
    """X of 64 MB: among the slab plans a power-law matrix gets slabs far beyond the L2 (its popular
    columns stay cached), a uniform one slabs of at most 6 MiB; both plans give the right product.
    Among the row-block plans both get 8 and 11 steps: the L2 asks for 13 and 21, but a block has 58,600 nonzeros and
    a step wants 7,000 (skewed columns) or 5,000 (even).  Left to choose, the library gives both a sweep plan (X of
    64 MB, nothing near the diagonal)."""
    K = 16
    rp, ci, val, X = workload(pkg, spec, K)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, K, rowblock="off", sweep="off")
    i = plan.info
    slab_bytes = i.slab_cols * K * 4
    assert i.num_slabs > 1 and i.hot_rows == 0
    assert (slab_bytes > (8 << 20)) == big_slabs and (big_slabs or slab_bytes <= (6 << 20) + 4096)
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    plan.close()
    blocks = pkg.spmm.Plan(csr, K, sweep="off")
    assert blocks.info.rowblock_steps == (8 if big_slabs else 11) and blocks.info.rowblock_blocks == 1024
    check_fp32(blocks.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    blocks.close()
    auto = pkg.spmm.Plan(csr, K)
    assert auto.info.sweep_panels == 512 and auto.info.sweep_tiles == 1 and auto.info.rowblock_steps == 0
    check_fp32(auto.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    auto.close()


@pytest.mark.parametrize("K", [16, 32, 64, 128, 256])
def test_rmat_config_full_size(pkg, orc, dev, K):
    # config 4: R-MAT scale 20, edge factor 16, deduplicated; the whole K sweep
    rp, ci, val, X = workload(pkg, pkg.graphs.CONFIG_SPECS["rmat_s20"], K)
    assert rp.size - 1 == 1 << 20
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    # The library's choice: a sweep plan, one round of 256 panels for 64-byte rows (2,444 accumulator rows each), two
    # rounds for the 128-byte column tiles of the wider rows (the longest row, a panel's share and more, cut into
    # sub-rows), one pass per tile.
    plan = pkg.spmm.Plan(csr, K)
    i = plan.info
    assert i.sweep_panels == (256 if K == 16 else 512) and i.sweep_tiles == max(1, K // 32) and i.sweep_lanes == (4 if K == 16 else 8)
    assert i.sweep_split_rows == (0 if K == 16 else 1) and i.sweep_slots <= 1.06 * ci.size
    # the other kinds of plan, which the library built for this matrix before it had sweep plans
    other = pkg.spmm.Plan(csr, K, sweep="off")
    # K = 64, X of 256 MiB (beyond the last-level cache): the 10 MiB of busiest columns stay plain gathers, the rest
    # is gathered with the streaming hint.  K = 128 and 256: 8-lane groups and one pass per 128 bytes of row pitch.
    if K == 16:
        # a row-block plan: 1,280 blocks (1,024 blocks of 1,024 rows would put 6 % of the nonzeros into the first)
        # of 12,600 nonzeros on average, which is worth one step
        assert other.info.rowblock_steps == 1 and other.info.rowblock_blocks == 1280
        slabs = pkg.spmm.Plan(csr, K, rowblock="off", sweep="off")
        assert slabs.info.rowblock_steps == 0 and slabs.info.num_slabs == 1 and slabs.info.threads_per_wave == 16
        check_fp32(slabs.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
        slabs.close()
    else:
        assert other.info.sweep_panels == 0 and other.info.num_slabs == 1 and (other.info.resident_cols > 0) == (K == 64)
        assert other.info.resident_cols == 0 or other.info.resident_nnz > 0.4 * ci.size
        assert other.info.threads_per_wave == (8 if K >= 128 else 64 // (K // 4)) and (K < 128 or other.info.cost == 64)
    check_fp32(other.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    other.close()
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    sched = pkg.spmm.generate_mp_sched(csr.row_ptr, csr.nnz)
    Yc = pkg.spmm.spmm_merge_path(csr, d_X, sched, out=torch.full_like(d_X, float("nan")))
    check_fp32(Yc.cpu().numpy(), ref, scale, rel_elem=False)
    if K in (16, 64):
        loops = cpu_fp32_loops(orc, rp, ci, val, X, sched.P)
        for Yg in (Y, Yc):
            check_against_cpu_fp32_loops(loops, ref, Yg.cpu().numpy())


@pytest.mark.parametrize("K", [24, 48])
def test_rmat_full_size_widths_that_leave_lanes_idle(pkg, orc, dev, K):
    # R-MAT scale 20 at widths between the benchmark's: 96-byte rows (one tile of 8 lanes, two of them idle) and
    # 192-byte rows (two tiles, half of the second idle); the library's choice is a sweep plan for both
    rp, ci, val, X = workload(pkg, pkg.graphs.CONFIG_SPECS["rmat_s20"], K)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    plan = pkg.spmm.Plan(csr, K)
    i = plan.info
    assert i.sweep_panels == 512 and i.sweep_lanes == 8 and i.sweep_tiles == (K * 4 + 127) // 128
    Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
    torch.cuda.synchronize()
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    other = pkg.spmm.Plan(csr, K, sweep="off")
    assert other.info.sweep_panels == 0
    check_fp32(other.spmm(d_X).cpu().numpy(), ref, scale, rel_elem=False)
    # the same bits from the plan built with the passes over the nonzeros on the host
    host = pkg.spmm.Plan(csr, K, host_build=True)
    assert torch.equal(host.spmm(d_X), Y)
    for pl in (plan, other, host):
        pl.close()


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
    # the library's choice: a sweep plan (fp32 sums of a 128-byte row of halves take 256 bytes of LDS: panels of about
    # 620 accumulator rows, many rounds of them); the slab plan with resident columns that it built before
    plan = pkg.spmm.Plan(csr, K)
    assert plan.info.sweep_panels >= 3584 and plan.info.sweep_lanes == 8 and plan.info.sweep_tiles == 1
    assert plan.info.sweep_acc_rows <= 632 and plan.info.sweep_split_rows > 0
    slab = pkg.spmm.Plan(csr, K, sweep="off")
    assert slab.info.resident_cols == (10 << 20) // 128 and slab.info.resident_nnz > 0.6 * ci.size
    for pl in (plan, slab):
        Y = pl.spmm(d_X, out=torch.full_like(d_X, float("nan")))
        torch.cuda.synchronize()
        Yh = Y.cpu().numpy().astype(np.float64)
        err = np.abs(Yh - ref)
        assert np.isfinite(Yh).all()
        assert (err <= 2e-2 * np.abs(ref) + 2e-5 * scale + 1e-6).all()      # the stated bar
        assert (err <= 2.0 ** -10 * np.abs(ref) + 1e-5 * scale + 1e-7).all()  # one half rounding
    slab.close()
    sched = pkg.spmm.generate_mp_sched(csr.row_ptr, csr.nnz)
    Yc = pkg.spmm.spmm_merge_path(csr, d_X, sched).cpu().numpy().astype(np.float64)
    assert (np.abs(Yc - ref) <= 2.0 ** -10 * np.abs(ref) + 1e-5 * scale + 1e-7).all()
