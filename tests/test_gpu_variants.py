"""fp16 variant, row_wise and nz_splitting comparison kernels, on the GPU,
against the oracle (fp64 row loop; row ranges and neighbour groups of the
reference restated in oracle/mp_oracle.c)."""
import numpy as np
import pytest
import torch

from gpu_util import check_fp16, check_fp32, make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("K", [8, 16, 20, 28, 32, 64, 100, 128, 256])  # 1, 4 (K = 16 .. 28) or 8 columns per lane
def test_fp16_against_oracle(pkg, orc, dev, K):
    rng = np.random.default_rng(K)
    n = 700
    rp, ci = random_csr(rng, n, 40, hub_rows=[(5, 650), (699, 300)])
    val = rng.random(ci.size).astype(np.float16)
    X = (rng.random((n, K)) * 2 - 1).astype(np.float16)
    ref, scale = orc.spmm_f64_f16in(rp, ci, val, X, want_abs=True)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    for cost in (8, 64):
        sched = pkg.spmm.generate_mp_sched(csr.row_ptr, csr.nnz, cost=cost)
        Y = pkg.spmm.spmm_merge_path(csr, d_X, sched, out=torch.full_like(d_X, float("nan")))
        torch.cuda.synchronize()
        assert Y.dtype == torch.float16
        check_fp16(Y.cpu().numpy(), ref, scale)
        for tiling, sb in (("off", 0), ("force", 128 * K * 2)):
            plan = pkg.spmm.Plan(csr, K, cost=cost, tiling=tiling, slab_bytes=sb)
            Yp = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
            torch.cuda.synchronize()
            check_fp16(Yp.cpu().numpy(), ref, scale)
            plan.close()


def test_fp16_rmat_reduced(pkg, orc, dev):
    # benchmark configuration 5 at reduced scale: R-MAT, half values / features, K = 64
    g = pkg.graphs
    rp, ci, _ = g.generate("rmat:scale=17,ef=16,a=0.57,b=0.19,c=0.19", seed=1)
    n, K = rp.size - 1, 64
    val = g.fill_uniform_f16(ci.size, 11, 0.0, 1.0)
    X = g.fill_uniform_f16(n * K, 13, -1.0, 1.0).reshape(n, K)
    ref, scale = orc.spmm_f64_f16in(rp, ci, val, X, want_abs=True)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    plan = pkg.spmm.Plan(csr, K)
    Y = plan.spmm(d_X)
    torch.cuda.synchronize()
    check_fp16(Y.cpu().numpy(), ref, scale)
    again = plan.spmm(d_X)
    assert torch.equal(Y, again)


def test_fp16_accumulates_in_fp32(pkg, dev):
    # 4096 terms of 1.0 * 1.0: an fp16 running sum would stall at 2048
    n, K = 4096, 32
    rp = np.concatenate([[0], np.full(n, n)]).astype(np.int32)  # row 0 holds every column
    ci = np.arange(n, dtype=np.int32)
    csr = make_csr(pkg, dev, rp, ci, np.ones(n, dtype=np.float16))
    X = torch.ones(n, K, dtype=torch.float16, device=dev)
    sched = pkg.spmm.generate_mp_sched(csr.row_ptr, n, cost=64)
    Y = pkg.spmm.spmm_merge_path(csr, X, sched)
    assert (Y[0] == 4096).all() and (Y[1:] == 0).all()


@pytest.mark.parametrize("K", [3, 16, 32, 48, 128])
def test_row_wise(pkg, orc, dev, K):
    rng = np.random.default_rng(K)
    n = 1000
    rp, ci = random_csr(rng, n, 30, hub_rows=[(17, 900)])
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    for num_waves in (1, 7, 64, 1000, 5000):
        Y = pkg.spmm.run_spmm_row_wise(csr, d_X, num_waves, out=torch.full_like(d_X, float("nan")))
        torch.cuda.synchronize()
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
    assert torch.equal(Y, pkg.spmm.run_spmm_row_wise(csr, d_X, 5000))


@pytest.mark.parametrize("part_size", [1, 4, 32, 1000])
def test_nz_splitting_groups_bit_exact(pkg, orc, dev, part_size):
    rng = np.random.default_rng(part_size)
    for n in (1, 50, 3000):
        rp, ci = random_csr(rng, n, 70, hub_rows=[(n // 2, n)] if n > 1 else ())
        (d_rp,) = to_dev(dev, rp)
        parts = pkg.spmm.build_part(d_rp, int(rp[-1]), part_size)
        pp, pn = orc.build_part(part_size, rp)
        assert parts.num_parts == orc.calculate_part_num(part_size, rp) == pn.size
        assert np.array_equal(parts.part_ptr.cpu().numpy(), pp)
        assert np.array_equal(parts.part2node.cpu().numpy(), pn)


@pytest.mark.parametrize("K", [5, 16, 64, 256])
def test_nz_splitting_spmm(pkg, orc, dev, K):
    rng = np.random.default_rng(K)
    n = 800
    rp, ci = random_csr(rng, n, 50, hub_rows=[(3, 700)])
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    for part_size in (1, 8, 32, 100):
        parts = pkg.spmm.build_part(csr.row_ptr, csr.nnz, part_size)
        out = torch.full_like(d_X, float("nan"))
        for _ in range(2):  # Y is zeroed by every call, not accumulated across repeats
            Y = pkg.spmm.spmm_nz_splitting(csr, d_X, parts, out=out)
        torch.cuda.synchronize()
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)


def test_large_scan_of_groups(pkg, orc, dev):
    # more rows than one scan segment (1024 * 2048) holds per pass
    n = (1 << 21) + 12345
    rng = np.random.default_rng(9)
    deg = rng.integers(0, 4, size=n)
    rp = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    (d_rp,) = to_dev(dev, rp)
    parts = pkg.spmm.build_part(d_rp, int(rp[-1]), 2)
    pp, pn = orc.build_part(2, rp)
    assert np.array_equal(parts.part_ptr.cpu().numpy(), pp)
    assert np.array_equal(parts.part2node.cpu().numpy(), pn)


@pytest.mark.parametrize("mode", ["product", "gcn"])
def test_degree_values(pkg, orc, dev, mode):
    """mps_degree_values_*: the reference's implicit weight deg(row) * deg(col)
    (src/MergePathSpMM.cu:183-185,450,459) as an array; bit-exact for the
    product (fp32 and half), one ulp for 1/sqrt."""
    g = pkg.graphs
    rp, ci, _ = g.generate("chunglu:n=6000,nnz=300000,gamma=2.1,dmax=5000", seed=9)
    # plus two hub rows that point at each other: 4097 * 4099 needs 25 bits, one fp32 rounding
    n = rp.size - 1
    hub = [np.r_[n + 1, np.arange(0, 4096)], np.r_[n, np.arange(0, 4098)]]
    ci = np.concatenate([ci] + hub).astype(np.int32)
    rp = np.concatenate([rp, [rp[-1] + 4097, rp[-1] + 4097 + 4099]]).astype(np.int32)
    d_rp, d_ci = to_dev(dev, rp, ci)
    for dtype, tdt in ((np.float32, torch.float32), (np.float16, torch.float16)):
        got = pkg.spmm.degree_values(d_rp, d_ci, mode=mode, dtype=tdt).cpu().numpy()
        want = orc.degree_values(rp, ci, mode=mode, dtype=dtype)
        if mode == "product":
            assert np.array_equal(got, want)  # inf == inf where half overflows
            if dtype == np.float16:
                assert np.isinf(want).any()
            else:
                assert (want > 2 ** 24).any()
        else:
            assert np.isfinite(got).all()
            ulp = np.spacing(np.abs(want).astype(dtype))
            assert (np.abs(got.astype(np.float64) - want.astype(np.float64)) <= ulp).all()


def test_spmm_with_degree_weights_and_unit_features(pkg, orc, dev):
    """The reference's setting (weights from degrees, all features 1.0): every
    output column is the row sum of the weights."""
    g = pkg.graphs
    rp, ci, _ = g.generate("rmat:scale=12,ef=8,a=0.57,b=0.19,c=0.19", seed=3)
    n, K = rp.size - 1, 16
    d_rp, d_ci = to_dev(dev, rp, ci)
    d_val = pkg.spmm.degree_values(d_rp, d_ci)
    val = orc.degree_values(rp, ci)
    X = np.ones((n, K), dtype=np.float32)
    csr = pkg.spmm.CsrDevice(d_rp, d_ci, d_val)
    plan = pkg.spmm.Plan(csr, K)
    (d_X,) = to_dev(dev, X)
    Y = plan.spmm(d_X).cpu().numpy()
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    check_fp32(Y, ref, scale, rel_elem=False)
    rows = np.repeat(np.arange(n), np.diff(rp))
    sums = np.bincount(rows, weights=val.astype(np.float64), minlength=n)
    assert np.allclose(Y[:, 0], sums, rtol=1e-5, atol=1e-6) and (Y == Y[:, :1]).all()
