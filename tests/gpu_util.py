"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def random_csr(rng, n, max_deg, p_empty=0.2, hub_rows=()):
    deg = rng.integers(0, max_deg + 1, size=n)
    deg[rng.random(n) < p_empty] = 0
    for r, d in hub_rows:
        deg[r] = d
    deg = np.minimum(deg, n)
    rp = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    parts = [np.sort(rng.choice(n, size=int(d), replace=False)) for d in deg if d > 0]
    ci = np.concatenate(parts) if parts else np.zeros(0, dtype=np.int64)
    return rp, ci.astype(np.int32)


def to_dev(dev, *arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in arrays]


def make_csr(pkg, dev, rp, ci, val):
    d_rp, d_ci, d_val = to_dev(dev, rp, ci, val)
    return pkg.spmm.CsrDevice(d_rp, d_ci, d_val)


def check_fp32(Y, ref, scale, rel_elem=True):
    """fp32 bar: |err| <= 1e-5 * |ref| + 1e-6 per element where the row has no
    heavy cancellation; always |err| <= 1e-5 * sum_j|a_ij x_jk| (the magnitude
    the rounding error of any summation order is relative to) and a norm-wise
    relative error <= 1e-5."""
    err = np.abs(Y.astype(np.float64) - ref)
    assert np.isfinite(Y).all()
    assert (err <= 1e-5 * scale + 1e-6).all(), "max err/scale %.3e" % float((err / (scale + 1e-30)).max())
    # tighter empirical guard: a dropped or doubled term is ~1e-1 of scale / degree
    assert (err <= 2e-6 * scale + 1e-6).all()
    nrm = np.linalg.norm(ref)
    if nrm > 0:
        assert np.linalg.norm(err) / nrm <= 1e-5
    if rel_elem:
        assert (err <= 1e-5 * np.abs(ref) + 1e-6).all()
    return float(err.max())


def check_fp16(Y, ref, scale):
    """fp16 bar: 2e-2 relative.  The device accumulates in fp32 and rounds once
    to half, so the error is half an ulp of the result (2^-11 relative) plus the
    fp32 accumulation error, far inside the bar; rows whose terms cancel are
    again measured against sum_j |a_ij x_jk|."""
    Y = Y.astype(np.float64)
    err = np.abs(Y - ref)
    assert np.isfinite(Y).all()
    assert (err <= 2e-2 * np.abs(ref) + 2e-2 * 1e-3 * scale + 1e-6).all()
    # what the arithmetic actually delivers: one half rounding of the result
    assert (err <= 2.0 ** -10 * np.abs(ref) + 1e-5 * scale + 1e-7).all()
