#!/usr/bin/env python3
"""Benchmark of the merge-path SpMM hot path on one MI355X.

A step is one SpMM launch (main kernel + carry-out fix-up) over a graph that
is already resident in HBM; the merge-path schedule is built once before the
loop, as the reference builds it once on the host
(src/MergePathSpMM.cu:192, repeat loop :231-243).

Prints ONE JSON line:  metric/value = GFLOP/s (2*nnz*K/t) of the default
workload (benchmark configuration 2: Chung-Lu power-law graph, fp32, K=16), plus
  roofline      algorithmic bytes / average duration of the main kernel,
                against the 8 TB/s HBM peak
  cpu_baseline  the oracle's multithreaded fp32 CSR SpMM on the host cores
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

PEAK_HBM_GBS = 8000.0

# HBM bytes per launch of the main kernel, from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised in
# profiles/mp_spmm_kernel_chunglu_233k_f32_k16.md (FETCH_SIZE x 2.0 and WRITE_SIZE x 1.0, the factors the copy
# probe gives, profiles/hbm_copy_probe_fetch_write_calibration.md).  Keyed by (workload, layout); other
# configurations report null.  Key: (workload, layout, column slabs, cost, hot columns per slab).
MEASURED_TRAFFIC = {
    # cold + hot launch of the main kernel: FETCH_SIZE 380,316 + 181,283 KiB raw, WRITE_SIZE 82,068 + 77,505 KiB
    ("chunglu_233k_f32_k16", "plan", 5, 64, 1728): int((380316 + 181283) * 1024 * 2.0 + (82068 + 77505) * 1024 * 1.0),
}

WORKLOADS = {
    # name: (generator spec, K, dtype)
    "chunglu_233k_f32_k16": ("chunglu:n=232965,nnz=114600000,gamma=2.1,dmax=20000", 16, "f32"),
    "er_4096_f32_k16": ("er:n=4096,deg=8", 16, "f32"),
    "blockdiag_1178_f32_k16": ("blockdiag:blocks=1178,min=100,max=600,deg=5", 16, "f32"),
    "rmat_s20_f32_k16": ("rmat:scale=20,ef=16,a=0.57,b=0.19,c=0.19", 16, "f32"),
    "rmat_s20_f32_k32": ("rmat:scale=20,ef=16,a=0.57,b=0.19,c=0.19", 32, "f32"),
    "rmat_s20_f32_k64": ("rmat:scale=20,ef=16,a=0.57,b=0.19,c=0.19", 64, "f32"),
    "rmat_s20_f32_k128": ("rmat:scale=20,ef=16,a=0.57,b=0.19,c=0.19", 128, "f32"),
    "rmat_s20_f32_k256": ("rmat:scale=20,ef=16,a=0.57,b=0.19,c=0.19", 256, "f32"),
    "rmat_s22_f16_k64": ("rmat:scale=22,ef=16,a=0.57,b=0.19,c=0.19", 64, "f16"),
}


def algorithmic_bytes(n_rows, nnz, K, val_bytes, elem_bytes):
    """row_ptr + col_idx + val + dense in + dense out."""
    return 4 * (n_rows + 1) + 4 * nnz + val_bytes * nnz + 2 * elem_bytes * n_rows * K


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="chunglu_233k_f32_k16", choices=sorted(WORKLOADS))
    ap.add_argument("--spec", default="", help="generator spec overriding the workload's graph (experiments)")
    ap.add_argument("--k", type=int, default=0, help="feature width overriding the workload's K (experiments)")
    ap.add_argument("--dtype", default="", choices=["", "f32", "f16"], help="element type overriding the workload's (experiments)")
    ap.add_argument("--cost", type=int, default=0, help="merge items per partition (0 = library default)")
    ap.add_argument("--mode", default="auto", choices=["auto", "plain", "untiled", "tiled"],
                    help="plain = kernels on the CSR arrays as given, no plan; auto / untiled / tiled = with a plan "
                         "(column-slab tiling where it pays / never / always)")
    ap.add_argument("--hot", default="auto", choices=["auto", "off", "force"],
                    help="hot columns of a tiled plan (their rows of X in LDS): where they pay / never / always")
    ap.add_argument("--rowblock", default="auto", choices=["auto", "off", "force"],
                    help="row-block plan (rows summed in LDS, popular columns' rows of X in LDS tables): where the "
                         "library picks it / never / always")
    ap.add_argument("--rb-steps", type=int, default=0, help="steps (LDS tables) of a row-block plan (0 = library default)")
    ap.add_argument("--rb-table-rows", type=int, default=0, help="rows per LDS table of a row-block plan (0 = what fits)")
    ap.add_argument("--slab-bytes", type=int, default=0, help="slab size for tiling (0 = library default)")
    ap.add_argument("--tpw", type=int, default=0, help="partitions per wavefront (0 = full wavefront)")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--graph", action="store_true",
                    help="capture one step in a HIP graph and time replays (what a launch-bound caller would do)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and the result check")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported (no multi-GPU path exists)" % args.gpus)

    import numpy as np
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    pkg = entry.load_package()
    sp, g = pkg.spmm, pkg.graphs
    dev = torch.device("cuda:0")
    spec, K, dt = WORKLOADS[args.workload]
    if args.spec:
        spec, args.workload = args.spec, "custom"
    if args.k:
        K, args.workload = args.k, "custom"
    if args.dtype:
        dt, args.workload = args.dtype, "custom"
    f16 = dt == "f16"
    eb = 2 if f16 else 4

    t0 = time.time()
    rp, ci, max_deg = g.generate(spec, seed=args.seed)
    n, nnz = rp.size - 1, ci.size
    fill = g.fill_uniform_f16 if f16 else g.fill_uniform_f32
    val = fill(nnz, 11, 0.0, 1.0)
    X = fill(n * K, 13, -1.0, 1.0).reshape(n, K)
    gen_s = time.time() - t0

    csr = sp.CsrDevice(torch.from_numpy(rp).to(dev), torch.from_numpy(ci).to(dev), torch.from_numpy(val).to(dev))
    d_X = torch.from_numpy(X).to(dev)
    d_Y = torch.full_like(d_X, float("nan"))
    csr.validate()
    cost = args.cost if args.cost > 0 else sp.default_cost(n, nnz, K, eb)
    plan = None
    if args.mode != "plain":
        tiling = {"auto": "auto", "untiled": "off", "tiled": "force"}[args.mode]
        plan_kw = dict(cost=cost, threads_per_wave=args.tpw, tiling=tiling, slab_bytes=args.slab_bytes, hot=args.hot,
                       rowblock=args.rowblock, rowblock_steps=args.rb_steps, rowblock_table_rows=args.rb_table_rows)
        plan = sp.Plan(csr, K, **plan_kw)
        P = plan.info.num_partitions
    else:
        sched = sp.generate_mp_sched(csr.row_ptr, nnz, cost=cost)
        P = sched.P
    torch.cuda.synchronize()
    PH = pkg._cabi
    tiled = plan is not None and plan.info.num_slabs > 1

    def step(phases=None):
        if plan is not None:
            plan.spmm(d_X, out=d_Y, phases=phases)
        else:
            sp.spmm_merge_path(csr, d_X, sched, threads_per_wave=args.tpw, out=d_Y, phases=phases)

    for _ in range(args.warmup):
        step()
    timed_step = step
    if args.graph:
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        hip_graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(hip_graph):
            step()
        timed_step = hip_graph.replay
        for _ in range(args.warmup):
            timed_step()
    # ---- timed region: exactly `steps` steps, inputs already in HBM ----------
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    w0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        timed_step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - w0) * 1e3
    ms_per_step = e0.elapsed_time(e1) / args.steps

    # ---- per-kernel durations over the same number of steps (events on the launch stream)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    for a, b, c, d in evs:
        a.record()
        step(PH.MPS_PHASE_MAIN)
        b.record()
        step(PH.MPS_PHASE_FIXUP)
        c.record()
        if tiled:
            step(PH.MPS_PHASE_REDUCE)
        d.record()
    torch.cuda.synchronize()
    main_ms = sum(a.elapsed_time(b) for a, b, _, _ in evs) / args.steps
    fix_ms = sum(b.elapsed_time(c) for _, b, c, _ in evs) / args.steps
    red_ms = sum(c.elapsed_time(d) for _, _, c, d in evs) / args.steps

    # preprocessing time (once per matrix, not part of a step)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    if plan is not None:
        sp.Plan(csr, K, **plan_kw).close()
    else:
        sp.generate_mp_sched(csr.row_ptr, nnz, cost=cost)
    torch.cuda.synchronize()
    plan_ms = (time.perf_counter() - t1) * 1e3

    hot_on = plan is not None and plan.info.hot_rows > 0
    flops = 2.0 * nnz * K
    b_alg = algorithmic_bytes(n, nnz, K, eb, eb)
    gflops = flops / (ms_per_step * 1e6)
    achieved = b_alg / (main_ms * 1e6)

    out = {
        "metric": "SpMM GFLOP/s (2*nnz*K/t), merge-path CSR x row-major dense",
        "value": round(gflops, 2),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dt,
        "data": "synthetic (seeded generator, values U[0,1), features U[-1,1))",
        "launch": "one HIP graph replay per step" if args.graph else "kernel launches per step",
        "config": {"workload": args.workload, "spec": spec, "n_rows": int(n), "nnz": int(nnz), "K": K,
                   "max_row_degree": int(max_deg), "cost": cost, "partitions": P,
                   "threads_per_wave": args.tpw or g.max_threads_per_wave(K, eb), "seed": args.seed,
                   "layout": "plain CSR, no plan" if plan is None else
                   ("row-block plan: %d blocks, %d steps x %d table rows, %.1f %% of the nonzeros from LDS, %.0f MB"
                    % (plan.info.rowblock_blocks, plan.info.rowblock_steps, plan.info.rowblock_table_rows,
                       100.0 * plan.info.hot_nnz / max(nnz, 1), plan.info.device_bytes / 1e6))
                   if plan.info.rowblock_steps > 0 else
                   ("plan: %d column slab(s) of %d, sliced, %.0f MB" % (plan.info.num_slabs, plan.info.slab_cols,
                                                                       plan.info.device_bytes / 1e6)) +
                   ("" if plan is None or plan.info.hot_rows == 0 else
                    ", %d hot columns per slab in LDS (%.1f %% of the nonzeros)"
                    % (plan.info.hot_rows, 100.0 * plan.info.hot_nnz / max(nnz, 1)))},
        "gbs_algorithmic_per_step": round(b_alg / (ms_per_step * 1e6), 2),
        "hbm_fraction_per_step": round(b_alg / (ms_per_step * 1e6) / PEAK_HBM_GBS, 4),
        "kernel_ms": {"mp_spmm_kernel": round(main_ms, 5), "mp_fixup_kernel": round(fix_ms, 5),
                      "tile_reduce_kernel": round(red_ms, 5),
                      "preprocessing, host wall time (once per matrix)": round(plan_ms, 3)},
        "wall_ms_per_step": round(wall_ms / args.steps, 5),
        "roofline": {"bound": "hbm", "kernel": "mp_spmm_kernel" + (" (hot + cold launch)" if hot_on else ""), "achieved": round(achieved, 2), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 4),
                     "traffic": MEASURED_TRAFFIC.get((args.workload, "plan" if plan is not None else "plain",
                                                      plan.info.num_slabs if plan is not None else 1, cost,
                                                      plan.info.hot_rows if plan is not None else 0)),
                     "algorithmic_bytes": int(b_alg)},
        "host_generate_s": round(gen_s, 2),
    }

    if not args.no_cpu:
        # CPU baseline leg: the oracle's multithreaded fp32 CSR x dense loop on
        # this box's host cores, bounded to a few passes over the same workload.
        orc = entry.load_oracle()
        threads = min(16, orc.max_threads(), os.cpu_count() or 1)
        val32 = val.astype(np.float32) if f16 else val
        X32 = X.astype(np.float32) if f16 else X
        Yc = np.empty((n, K), dtype=np.float32)
        orc.spmm_f32_mt(rp, ci, val32, X32, threads=threads, out=Yc)  # warm
        passes, spent = 0, 0.0
        while passes < 20 and spent < 10.0:
            c0 = time.perf_counter()
            orc.spmm_f32_mt(rp, ci, val32, X32, threads=threads, out=Yc)
            spent += time.perf_counter() - c0
            passes += 1
        cpu_s = spent / passes
        out["cpu_baseline"] = {"value": round(flops / cpu_s / 1e9, 3), "unit": "GFLOP/s", "cores": threads,
                               "kind": "port", "sample": "%d full passes over the same workload, %.3f s each"
                               % (passes, cpu_s)}
        Yg = d_Y.float().cpu().numpy()
        err = np.abs(Yg.astype(np.float64) - Yc.astype(np.float64))
        out["check_vs_cpu_fp32"] = {"max_abs_diff": float(err.max()),
                                    "rel_fro": float(np.linalg.norm(err) / max(np.linalg.norm(Yc), 1e-30))}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
