"""Column-slab tiled merge-path SpMM: the tiled arrays are a permutation of
the CSR (checked against a numpy restatement of the slab-major order), and the
result meets the same bar against the oracle's fp64 row loop."""
import numpy as np
import pytest
import torch

from gpu_util import check_fp32, make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu


def slab_major_reference(rp, ci, num_slabs, slab_cols):
    """(vrow_ptr, perm) of the slab-major order: virtual row s*n + r holds row r's
    nonzeros with s*slab_cols <= col < (s+1)*slab_cols, in their original order."""
    n = rp.size - 1
    rows = np.repeat(np.arange(n, dtype=np.int64), np.diff(rp))
    slab = np.minimum(ci.astype(np.int64) // slab_cols, num_slabs - 1)
    v = slab * n + rows
    perm = np.argsort(v, kind="stable")
    counts = np.bincount(v, minlength=num_slabs * n)
    vrp = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    return vrp, perm.astype(np.int32)


@pytest.mark.parametrize("num_slabs,slab_cols", [(1, 512), (2, 256), (4, 128), (7, 74), (64, 8)])
def test_tile_build_matches_numpy(pkg, dev, num_slabs, slab_cols):
    rng = np.random.default_rng(num_slabs)
    n = 500
    rp, ci = random_csr(rng, n, 40, hub_rows=[(3, 450), (499, 300)])
    val = rng.random(ci.size).astype(np.float32)
    csr = make_csr(pkg, dev, rp, ci, val)
    t = pkg.spmm.build_tiles(csr, 16, cost=16, num_slabs=num_slabs, slab_cols=slab_cols)
    torch.cuda.synchronize()
    vrp, perm = slab_major_reference(rp, ci, num_slabs, slab_cols)
    assert np.array_equal(t.vrow_ptr.cpu().numpy(), vrp)
    assert np.array_equal(t.perm.cpu().numpy()[: ci.size], perm)
    assert np.array_equal(t.col_tiled.cpu().numpy()[: ci.size], ci[perm])
    assert np.array_equal(t.val_tiled.cpu().numpy()[: ci.size], val[perm])
    # new values flow through set_values
    val2 = rng.random(ci.size).astype(np.float32)
    t.set_values(torch.from_numpy(val2).to(dev))
    assert np.array_equal(t.val_tiled.cpu().numpy()[: ci.size], val2[perm])


def test_unsorted_rows_are_refused(pkg, dev):
    rp = np.array([0, 3, 5], dtype=np.int32)
    ci = np.array([2, 1, 0, 0, 1], dtype=np.int32)  # row 0 decreasing
    csr = make_csr(pkg, dev, rp, ci, np.ones(5, dtype=np.float32))
    with pytest.raises(pkg.MpsError) as e:
        pkg.spmm.build_tiles(csr, 16, cost=4, num_slabs=2, slab_cols=64)
    assert e.value.status == pkg._cabi.MPS_ERR_UNSORTED
    # a decrease exactly at a row boundary is fine, and so are repeated ids
    ci_ok = np.array([0, 1, 1, 0, 1], dtype=np.int32)
    csr = make_csr(pkg, dev, rp, ci_ok, np.ones(5, dtype=np.float32))
    assert pkg.spmm.build_tiles(csr, 16, cost=4, num_slabs=2, slab_cols=64) is not None


@pytest.mark.parametrize("K", [4, 16, 20, 64, 256])
def test_tiled_spmm_against_oracle(pkg, orc, dev, K):
    rng = np.random.default_rng(100 + K)
    n = 900
    rp, ci = random_csr(rng, n, 60, hub_rows=[(0, 800), (450, 777), (899, 600)])
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    for num_slabs, slab_cols, cost in ((3, 320, 32), (8, 128, 128), (1, 960, 16), (15, 64, 7)):
        t = pkg.spmm.build_tiles(csr, K, cost=cost, num_slabs=num_slabs, slab_cols=slab_cols)
        out = torch.full_like(d_X, float("nan"))
        Y = pkg.spmm.spmm_merge_path_tiled(t, d_X, out=out)
        torch.cuda.synchronize()
        check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        again = pkg.spmm.spmm_merge_path_tiled(t, d_X, out=torch.empty_like(d_X))
        assert torch.equal(Y, again)  # deterministic


def test_tile_shape_heuristic(pkg):
    sp = pkg.spmm
    # config 2: X = 14.9 MB, ~492 nonzeros per row -> 8 slabs of ~2 MiB
    ns, sc = sp.tile_shape(232965, 114604189, 16, 4)
    assert ns == 8 and sc * 16 * 4 <= (2 << 20) + 64 * 64 and ns * sc >= 232965
    assert sp.tile_shape(4096, 32731, 16, 4)[0] == 1  # X fits in L2
    assert sp.tile_shape(1048576, 16086273, 16, 4)[0] == 1  # too few nonzeros per row and slab


def test_power_law_graph_tiled_vs_plain(pkg, orc, dev):
    g = pkg.graphs
    rp, ci, _ = g.generate("chunglu:n=100000,nnz=20000000,gamma=2.1,dmax=9000", seed=2)
    n, K = rp.size - 1, 16
    val = g.fill_uniform_f32(ci.size, 11, 0.0, 1.0)
    X = g.fill_uniform_f32(n * K, 13, -1.0, 1.0).reshape(n, K)
    ref, scale = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    t = pkg.spmm.build_tiles(csr, K, cost=128)
    assert t is not None and t.num_slabs == 4
    Y = pkg.spmm.spmm_merge_path_tiled(t, d_X)
    torch.cuda.synchronize()
    check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
