"""Merge-path partitioner on the GPU, bit-exact against the oracle
(src/MergePathSpMM.cu:280-385 restated in oracle/mp_oracle.c)."""
import numpy as np
import pytest
import torch

from gpu_util import random_csr, to_dev

pytestmark = pytest.mark.gpu


def gpu_coords(pkg, dev, rp, nnz, P):
    (d_rp,) = to_dev(dev, rp)
    sched = pkg.spmm.generate_mp_sched(d_rp, nnz, P=P)
    torch.cuda.synchronize()
    return sched, d_rp


def test_worked_examples(pkg, orc, dev):
    import json, os
    with open(os.path.join(os.path.dirname(__file__), "golden", "worked_examples.json")) as f:
        golden = json.load(f)
    for case in golden["coords"]:
        rp = np.array(case["row_ptr"], dtype=np.int32)
        sched, _ = gpu_coords(pkg, dev, rp, int(rp[-1]), case["P"])
        assert sched.coord_x.cpu().tolist() == case["x"]
        assert sched.coord_y.cpu().tolist() == case["y"]
    for case in golden["sched"]:
        rp = np.array(case["row_ptr"], dtype=np.int32)
        sched, d_rp = gpu_coords(pkg, dev, rp, int(rp[-1]), case["P"])
        legacy = sched.legacy_arrays(d_rp)
        for name in orc.SCHED_FIELDS:
            assert legacy[name].cpu().tolist() == case[name], name


def test_random_csrs_bit_exact(pkg, orc, dev):
    rng = np.random.default_rng(2024)
    for trial in range(40):
        n = int(rng.integers(1, 400))
        rp, ci = random_csr(rng, n, int(rng.integers(1, 60)), hub_rows=[(int(rng.integers(0, n)), n // 2)])
        nnz = int(rp[-1])
        for P in (1, 3, int(rng.integers(4, 200)), 1024, n + 1 + nnz + 17):
            sched, d_rp = gpu_coords(pkg, dev, rp, nnz, P)
            xs, ys = orc.partition_coords(rp, nnz, P)
            assert np.array_equal(sched.coord_x.cpu().numpy(), xs), (trial, P)
            assert np.array_equal(sched.coord_y.cpu().numpy(), ys), (trial, P)
            legacy = sched.legacy_arrays(d_rp)
            want = orc.generate_mp_sched(rp, nnz, P)
            for name in orc.SCHED_FIELDS:
                assert np.array_equal(legacy[name].cpu().numpy(), want[name]), (trial, P, name)


@pytest.mark.parametrize("spec,cost", [
    ("er:n=4096,deg=8", 32),
    ("er:n=4096,deg=8", 7),
    ("blockdiag:blocks=1178,min=100,max=600,deg=5", 64),
    ("rmat:scale=16,ef=16,a=0.57,b=0.19,c=0.19", 128),
    ("chunglu:n=30000,nnz=3000000,gamma=2.1,dmax=5000", 128),
])
def test_benchmark_graphs_bit_exact(pkg, orc, dev, spec, cost):
    rp, ci, _ = pkg.graphs.generate(spec, seed=1)
    n, nnz = rp.size - 1, ci.size
    P = pkg.graphs.num_partitions(n, nnz, cost)
    assert P == orc.num_partitions(n, nnz, cost)
    sched, d_rp = gpu_coords(pkg, dev, rp, nnz, P)
    xs, ys = orc.partition_coords(rp, nnz, P)
    assert np.array_equal(sched.coord_x.cpu().numpy(), xs)
    assert np.array_equal(sched.coord_y.cpu().numpy(), ys)
    legacy = sched.legacy_arrays(d_rp)
    want = orc.generate_mp_sched(rp, nnz, P)
    for name in orc.SCHED_FIELDS:
        assert np.array_equal(legacy[name].cpu().numpy(), want[name]), name


def test_empty_matrix_and_no_nonzeros(pkg, orc, dev):
    for rp in (np.array([0], dtype=np.int32), np.zeros(6, dtype=np.int32)):
        sched, _ = gpu_coords(pkg, dev, rp, 0, 5)
        xs, ys = orc.partition_coords(rp, 0, 5)
        assert np.array_equal(sched.coord_x.cpu().numpy(), xs)
        assert np.array_equal(sched.coord_y.cpu().numpy(), ys)


def test_validate(pkg, dev):
    rp = np.array([0, 2, 3, 4], dtype=np.int32)
    ci = np.array([1, 2, 0, 1], dtype=np.int32)
    val = np.ones(4, dtype=np.float32)
    from gpu_util import make_csr
    make_csr(pkg, dev, rp, ci, val).validate()
    for bad_rp, bad_ci in ((np.array([0, 3, 2, 4], dtype=np.int32), ci), (rp, np.array([1, 2, 0, 3], dtype=np.int32)),
                           (np.array([1, 2, 3, 4], dtype=np.int32), ci), (rp, np.array([1, -1, 0, 1], dtype=np.int32))):
        with pytest.raises(pkg.MpsError) as e:
            make_csr(pkg, dev, bad_rp, bad_ci, val).validate()
        assert e.value.status == pkg._cabi.MPS_ERR_INVALID_CSR
