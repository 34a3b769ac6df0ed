"""Seeded random sweep over plans: matrix shape, row lengths, hub rows, K, dtype,
tiling, slab width, hot columns, cost and partitions per wavefront, each against
the oracle's fp64 row loop, and twice in a row for bit-identical results."""
import numpy as np
import pytest
import torch

from gpu_util import check_fp16, check_fp32, make_csr, random_csr, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_plans_against_oracle(pkg, orc, dev, seed):
    rng = np.random.default_rng(seed)
    for case in range(40):
        n = int(rng.integers(1, 4000))
        max_deg = int(rng.choice([1, 3, 12, 60]))
        hubs = [(int(rng.integers(0, n)), int(rng.integers(1, n + 1))) for _ in range(int(rng.integers(0, 3)))]
        rp, ci = random_csr(rng, n, max_deg, hub_rows=hubs)
        dt = np.float16 if rng.integers(0, 2) else np.float32
        K = int(rng.choice([16, 16, 16, 32, 8, 20, 64]))
        val = rng.random(ci.size).astype(dt)
        X = (rng.random((n, K)) * 2 - 1).astype(dt)
        tiling = str(rng.choice(["off", "force", "force", "auto"]))
        slab_cols = int(rng.choice([64, 128, 512, 2048]))
        hot = str(rng.choice(["auto", "off", "force"]))
        cost = int(rng.choice([1, 3, 7, 16, 32, 64, 128, 300]))
        max_tpw = pkg.graphs.max_threads_per_wave(K, val.itemsize)
        tpw = int(rng.choice([0, 1, max_tpw, max(1, max_tpw // 2)]))
        what = dict(seed=seed, case=case, n=n, nnz=int(ci.size), K=K, dtype=dt.__name__, tiling=tiling, slab_cols=slab_cols,
                    hot=hot, cost=cost, tpw=tpw, hubs=hubs)
        print(what, flush=True)  # names the case should a launch go wrong
        csr = make_csr(pkg, dev, rp, ci, val)
        plan = pkg.spmm.Plan(csr, K, cost=cost, threads_per_wave=tpw, tiling=tiling, slab_bytes=slab_cols * K * val.itemsize,
                             hot=hot)
        (d_X,) = to_dev(dev, X)
        Y = plan.spmm(d_X, out=torch.full_like(d_X, float("nan")))
        torch.cuda.synchronize()
        ref, scale = orc.spmm_f64(rp, ci, val.astype(np.float32), X.astype(np.float32), want_abs=True)
        if dt == np.float16:
            check_fp16(Y.cpu().numpy(), ref, scale)
        else:
            check_fp32(Y.cpu().numpy(), ref, scale, rel_elem=False)
        again = plan.spmm(d_X)
        torch.cuda.synchronize()
        assert torch.equal(Y, again), what
        plan.close()
