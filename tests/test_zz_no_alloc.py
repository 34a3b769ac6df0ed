"""mps_spmm_f32_static: the merge-path SpMM with its carry-out records in the library's own
device array (no allocation, no workspace argument) gives the bits of mps_spmm_f32."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu


def run_both(pkg, dev, rp, ci, val, X, cost):
    sp, C = pkg.spmm, pkg._cabi
    csr = make_csr(pkg, dev, rp, ci, val)
    (d_X,) = to_dev(dev, X)
    sched = sp.generate_mp_sched(csr.row_ptr, csr.nnz, cost=cost)
    Y_ref = sp.spmm_merge_path(csr, d_X, sched, out=torch.full_like(d_X, float("nan")))
    Y = torch.full_like(d_X, float("nan"))
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # device memory as the driver counts it (hipMemGetInfo): a hipMalloc inside the library would show here, which
    # torch's own allocator statistics would not; the call goes out twice so that anything a first call sets up
    # lazily (the address of the library's array) is not taken for an allocation of the second
    args = (vp(csr.row_ptr), vp(csr.col_idx), vp(csr.val), vp(d_X), vp(Y), csr.n_rows, csr.nnz, X.shape[1], sched.P,
            vp(sched.coord_x), vp(sched.coord_y), 0, stream)
    C.check(C.lib().mps_spmm_f32_static(*args), "mps_spmm_f32_static")
    torch.cuda.synchronize()
    Y.fill_(float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    free_before = torch.cuda.mem_get_info(dev)[0]
    C.check(C.lib().mps_spmm_f32_static(*args), "mps_spmm_f32_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.equal(Y, Y_ref)
    return sched.P


def test_static_scratch_entry_point_matches_the_workspace_one(pkg, dev):
    rng = np.random.default_rng(21)
    # two calls in a row, the second on a smaller input: it must not see the first one's records
    n1 = 6000
    rp1, ci1 = random_csr(rng, n1, 60, hub_rows=((7, 5000), (5999, 3000)))
    v1 = rng.random(ci1.size).astype(np.float32)
    X1 = (rng.random((n1, 16)) * 2 - 1).astype(np.float32)
    P1 = run_both(pkg, dev, rp1, ci1, v1, X1, cost=8)
    n2 = 700
    rp2, ci2 = random_csr(rng, n2, 30, hub_rows=((0, 650),))
    v2 = rng.random(ci2.size).astype(np.float32)
    X2 = (rng.random((n2, 16)) * 2 - 1).astype(np.float32)
    P2 = run_both(pkg, dev, rp2, ci2, v2, X2, cost=8)
    assert P2 < P1
    # other widths share the array
    X3 = (rng.random((n2, 64)) * 2 - 1).astype(np.float32)
    run_both(pkg, dev, rp2, ci2, v2, X3, cost=16)


def test_static_scratch_limit_is_reported(pkg, dev):
    C = pkg._cabi
    nbytes = ctypes.c_size_t()
    C.check(C.lib().mps_static_scratch_bytes(ctypes.byref(nbytes)), "mps_static_scratch_bytes")
    assert nbytes.value == 32 << 20
    # more partitions than the array holds records for: refused, nothing launched
    P = 40_000_000
    need = ctypes.c_size_t()
    C.check(C.lib().mps_spmm_workspace_bytes(P, 16, 0, 4, ctypes.byref(need)), "mps_spmm_workspace_bytes")
    assert need.value > nbytes.value
    one = torch.zeros(16, dtype=torch.int32, device=dev)
    vp = ctypes.c_void_p(one.data_ptr())
    rc = C.lib().mps_spmm_f32_static(vp, vp, vp, vp, vp, 1, 0, 16, P, vp, vp, 0, None)
    assert rc == C.MPS_ERR_WORKSPACE
