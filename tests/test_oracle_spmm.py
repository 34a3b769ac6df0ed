"""Pins the oracle's SpMM loops without a GPU: closed forms (identity matrix,
all-ones features), a library routine (scipy.sparse), and agreement between
the fp64 row loop and the reference-structured fp32 walk."""
import numpy as np
import pytest
import scipy.sparse as sps


def random_csr(rng, n, max_deg, p_empty=0.2):
    deg = rng.integers(0, max_deg + 1, size=n)
    deg[rng.random(n) < p_empty] = 0
    deg = np.minimum(deg, n)
    rp = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(n, size=d, replace=False)) for d in deg] + [np.zeros(0, int)])
    return rp, ci.astype(np.int32)


def test_identity_matrix(orc):
    n, K = 37, 5
    rp = np.arange(n + 1, dtype=np.int32)
    ci = np.arange(n, dtype=np.int32)
    val = np.ones(n, dtype=np.float32)
    X = np.random.default_rng(0).standard_normal((n, K)).astype(np.float32)
    assert np.array_equal(orc.spmm_f64(rp, ci, val, X), X.astype(np.float64))
    assert np.array_equal(orc.spmm_f32_mt(rp, ci, val, X, threads=3), X)
    assert np.array_equal(orc.spmm_mergepath_f32(rp, ci, val, X, 7), X)


def test_all_ones_features_give_row_sums(orc):
    rng = np.random.default_rng(1)
    rp, ci = random_csr(rng, 200, 30)
    val = rng.random(ci.size).astype(np.float32)
    X = np.ones((200, 4), dtype=np.float32)
    Y, A = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    rows = np.array([val[rp[i]:rp[i + 1]].astype(np.float64).sum() for i in range(200)])
    assert np.allclose(Y, rows[:, None], rtol=1e-14, atol=0)
    assert np.allclose(A, Y, rtol=1e-14)


@pytest.mark.parametrize("K", [1, 3, 16, 33])
def test_against_scipy(orc, K):
    rng = np.random.default_rng(K)
    n = 300
    rp, ci = random_csr(rng, n, 40)
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, K)) * 2 - 1).astype(np.float32)
    ref = sps.csr_matrix((val.astype(np.float64), ci, rp), shape=(n, n)) @ X.astype(np.float64)
    got = orc.spmm_f64(rp, ci, val, X)
    assert np.allclose(got, ref, rtol=1e-13, atol=1e-15)
    # scale output: |A| @ |X|
    _, A = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    ref_abs = sps.csr_matrix((np.abs(val.astype(np.float64)), ci, rp), shape=(n, n)) @ np.abs(X.astype(np.float64))
    assert np.allclose(A, ref_abs, rtol=1e-13, atol=1e-15)
    # fp32 loops agree with fp64 within fp32 rounding of the row's magnitude
    for Y32 in (orc.spmm_f32_mt(rp, ci, val, X, threads=4), orc.spmm_mergepath_f32(rp, ci, val, X, 13)):
        assert (np.abs(Y32 - ref) <= 1e-6 * ref_abs + 1e-30).all()


def test_mergepath_walk_handles_split_rows(orc):
    # one long row cut by many partitions, the first row longer than a partition
    # (the case the reference's zero sentinel loses), empty rows, partial last row
    rng = np.random.default_rng(3)
    deg = np.array([70, 0, 0, 1, 500, 0, 3, 29], dtype=np.int64)
    n = deg.size
    rp = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    ci = rng.integers(0, n, size=rp[-1]).astype(np.int32)
    val = rng.random(ci.size).astype(np.float32)
    X = (rng.random((n, 8)) * 2 - 1).astype(np.float32)
    ref, A = orc.spmm_f64(rp, ci, val, X, want_abs=True)
    for P in (1, 2, 5, 19, 64, 700):
        Y = orc.spmm_mergepath_f32(rp, ci, val, X, P)
        assert (np.abs(Y - ref) <= 1e-6 * A + 1e-30).all(), P
        assert (Y[deg == 0] == 0).all()


def test_half_inputs(orc):
    rng = np.random.default_rng(4)
    n, K = 120, 8
    rp, ci = random_csr(rng, n, 25)
    val = rng.random(ci.size).astype(np.float16)
    X = (rng.random((n, K)) * 2 - 1).astype(np.float16)
    got = orc.spmm_f64_f16in(rp, ci, val, X)
    ref = sps.csr_matrix((val.astype(np.float64), ci, rp), shape=(n, n)) @ X.astype(np.float64)
    assert np.allclose(got, ref, rtol=1e-13, atol=1e-15)
    # bit patterns: subnormal, one, max, -2
    for bits, want in ((0x0001, 2.0 ** -24), (0x3c00, 1.0), (0x7bff, 65504.0), (0xc000, -2.0), (0x0000, 0.0)):
        assert orc.lib().orc_half_to_double(bits) == want


def test_degree_values_hand_example(orc):
    # degrees 2, 1, 0, 3; weight of (r, c) = deg r * deg c (src/MergePathSpMM.cu:183-185,450,459)
    rp = np.array([0, 2, 3, 3, 6], dtype=np.int32)
    ci = np.array([1, 3, 0, 0, 1, 3], dtype=np.int32)
    assert orc.degree_values(rp, ci).tolist() == [2.0, 6.0, 2.0, 6.0, 3.0, 9.0]
    assert orc.degree_values(rp, ci, dtype=np.float16).tolist() == [2.0, 6.0, 2.0, 6.0, 3.0, 9.0]
    g = orc.degree_values(rp, ci, mode="gcn")
    want = [2 ** -0.5, 6 ** -0.5, 2 ** -0.5, 6 ** -0.5, 3 ** -0.5, 1 / 3]
    assert np.allclose(g, want, rtol=2e-7, atol=0) and g.dtype == np.float32


def test_degree_values_rounding_and_half_overflow(orc):
    # two hub rows that point at each other: 4097 * 4099 = 16,793,603 needs 25 bits -> one fp32 rounding
    n = 4100
    deg = np.zeros(n, dtype=np.int64)
    deg[0], deg[1] = 4097, 4099
    rp = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    ci = np.concatenate([np.r_[1, np.arange(2, 4098)], np.r_[0, np.arange(2, 4100)]]).astype(np.int32)
    w = orc.degree_values(rp, ci)
    assert w[0] == np.float32(16793603) and float(w[0]) in (16793602.0, 16793604.0)
    assert w[4097] == w[0] and w[1] == 0.0  # column 2 has degree 0
    h = orc.degree_values(rp, ci, dtype=np.float16)
    assert np.isinf(h[0]) and h[1] == 0.0  # half(4097) * half(4099) = 4096 * 4100 > 65504
    rp2 = np.array([0, 200, 400] + [400] * 198, dtype=np.int32)  # degrees 200, 200, then empty rows
    ci2 = np.concatenate([np.arange(200), np.arange(200)]).astype(np.int32)
    h2 = orc.degree_values(rp2, ci2, dtype=np.float16)
    assert h2[0] == 40000.0 and h2[1] == 40000.0 and h2[2] == 0.0  # 200 * 200 fits half
    g = orc.degree_values(rp2, ci2, mode="gcn")
    assert g[0] == np.float32(1.0) / np.float32(200.0) and g[2] == 0.0
