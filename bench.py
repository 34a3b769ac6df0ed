#!/usr/bin/env python3
"""Benchmark of the merge-path SpMM hot path on one MI355X.

A step is one product Y = A X over a graph that is already resident in HBM;
the per-matrix preprocessing (a plan) is built once before the loop, as the
reference builds its schedule once on the host (src/MergePathSpMM.cu:192,
repeat loop :231-243).

Prints ONE JSON line:  metric/value = GFLOP/s (2*nnz*K/t) of the default
workload (benchmark configuration 2: Chung-Lu power-law graph, fp32, K=16), plus
  roofline      algorithmic bytes / average duration of the dominant kernel,
                against the 8 TB/s HBM peak; traffic = HBM bytes per launch of
                that kernel from the counter runs summarised under profiles/
  cpu_baseline  the oracle's multithreaded fp32 CSR SpMM on the host cores
  configs       the other benchmark configurations, timed with the same loop
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

PEAK_HBM_GBS = 8000.0
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_by_plan.md")

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
HEADLINE = "chunglu_233k_f32_k16"
# the configurations of the benchmark besides the headline one, in its order (1, 3, 4 at five widths, 5)
OTHER_CONFIGS = ["er_4096_f32_k16", "blockdiag_1178_f32_k16", "rmat_s20_f32_k16", "rmat_s20_f32_k32",
                 "rmat_s20_f32_k64", "rmat_s20_f32_k128", "rmat_s20_f32_k256", "rmat_s22_f16_k64"]


def algorithmic_bytes(n_rows, nnz, K, val_bytes, elem_bytes):
    """row_ptr + col_idx + val + dense in + dense out."""
    return 4 * (n_rows + 1) + 4 * nnz + val_bytes * nnz + 2 * elem_bytes * n_rows * K


def plan_signature(workload, info):
    """What decides the HBM traffic of a plan's dominant kernel: the workload and the plan's shape."""
    if info is None:
        return "%s|csr" % workload
    if info.sweep_panels > 0:
        return "%s|sweep|panels=%d|tiles=%d|acc_rows=%d|piece=%d" % (workload, info.sweep_panels, info.sweep_tiles,
                                                                     info.sweep_acc_rows, info.sweep_piece)
    if info.rowblock_steps > 0:
        return "%s|rowblock|steps=%d|table_rows=%d|blocks=%d|cold_index_bits=%d" % (
            workload, info.rowblock_steps, info.rowblock_table_rows, info.rowblock_blocks, info.rowblock_cold_index_bits)
    return "%s|slabs=%d|cost=%d|tpw=%d|hot_rows=%d|resident_cols=%d" % (workload, info.num_slabs, info.cost,
                                                                        info.threads_per_wave, info.hot_rows, info.resident_cols)


def lines_read_once(w, info):
    """128-byte lines that a product of a row-block or sweep plan touches exactly once - the plan's entry streams and
    the rows of Y - and that therefore miss L2 by nature; None for the other kinds of plan, whose partial rows are
    written and read again."""
    if info is None or (info.sweep_panels == 0 and info.rowblock_steps == 0):
        return None
    streams = 8 * int(info.sweep_slots) * info.sweep_tiles if info.sweep_panels > 0 else int(info.device_bytes)
    return (streams + w.n * w.K * w.eb) // 128


def measured_counters(signature, with_requests=False, other_lines=None):
    """Counter readings for this plan shape from the table of counter runs under profiles/: HBM bytes per launch of the
    dominant kernel (FETCH_SIZE and WRITE_SIZE in KiB per dispatch, each scaled by what the same counter reads for a
    plain copy of known size), the L2 hit rate of that kernel (TCC_HIT / (TCC_HIT + TCC_MISS), all its requests: the
    gathers of rows of X, the sparse streams and the stores) and the summary they come from.  (None, None, None) when the
    table has no row for the signature; the hit rate is None for rows measured before it was collected."""
    none = (None, None, None, None) if with_requests else (None, None, None)
    try:
        text = open(TRAFFIC_TABLE).read()
    except OSError:
        return none
    for line in text.splitlines():
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        # | signature (its own '|' written as ';') | kernel | FETCH_SIZE KiB | fetch factor | WRITE_SIZE KiB | write factor |
        #   [TCC_HIT | TCC_MISS |] summary |
        if len(cells) in (7, 9) and cells[0].replace(";", "|").replace("`", "") == signature:
            try:
                fetch, ff, write, wf = float(cells[2]), float(cells[3]), float(cells[4]), float(cells[5])
                hit_rate = gather_rate = None
                if len(cells) == 9:
                    hits, misses = float(cells[6]), float(cells[7])
                    hit_rate = round(hits / (hits + misses), 4) if hits + misses > 0 else None
                    # the gathers of rows of X alone: all requests less the lines that are touched once (they miss)
                    if other_lines is not None and hits + misses > other_lines and misses >= other_lines:
                        gather_rate = round(hits / (hits + misses - other_lines), 4)
            except ValueError:
                continue
            found = (int((fetch * ff + write * wf) * 1024), hit_rate, "profiles/" + cells[-1].replace("`", ""))
            return found + (gather_rate,) if with_requests else found
    return none


def measured_traffic(signature):
    """(HBM bytes per launch of the dominant kernel, the summary under profiles/ it comes from) for a plan signature."""
    traffic, _, where = measured_counters(signature)
    return traffic, where


class Workload:
    """One benchmark configuration resident on the device."""

    def __init__(self, pkg, name, spec, K, dt, seed, torch, dev, values="uniform"):
        g, sp = pkg.graphs, pkg.spmm
        self.name, self.spec, self.K, self.dt = name, spec, K, dt
        self.f16 = dt == "f16"
        self.eb = 2 if self.f16 else 4
        t0 = time.time()
        self.rp, self.ci, self.max_deg = g.generate(spec, seed=seed)
        self.n, self.nnz = self.rp.size - 1, self.ci.size
        fill = g.fill_uniform_f16 if self.f16 else g.fill_uniform_f32
        self.X = fill(self.n * K, 13, -1.0, 1.0).reshape(self.n, K)
        d_rp, d_ci = torch.from_numpy(self.rp).to(dev), torch.from_numpy(self.ci).to(dev)
        if values == "uniform":
            self.val = fill(self.nnz, 11, 0.0, 1.0)
            d_val = torch.from_numpy(self.val).to(dev)
        else:
            # the reference's implicit edge weight (or the GCN norm) as an explicit array, made on the device
            d_val = sp.degree_values(d_rp, d_ci, mode="product" if values == "degree" else "gcn",
                                     dtype=torch.float16 if self.f16 else torch.float32)
            self.val = d_val.cpu().numpy()
        self.gen_s = time.time() - t0
        self.csr = sp.CsrDevice(d_rp, d_ci, d_val)
        self.d_X = torch.from_numpy(self.X).to(dev)
        self.d_Y = torch.full_like(self.d_X, float("nan"))
        self.csr.validate()
        self.flops = 2.0 * self.nnz * K
        self.b_alg = algorithmic_bytes(self.n, self.nnz, K, self.eb, self.eb)


def time_steps(torch, step, steps, warmup):
    """warmup untimed steps, then exactly `steps` steps between synchronisations; ms per step (HIP events)."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    w0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps, (time.perf_counter() - w0) * 1e3 / steps


def layout_text(w, plan):
    if plan is None:
        return "plain CSR, no plan"
    i = plan.info
    if i.sweep_panels > 0:
        return ("sweep plan: %d panels x %d column tile(s) of %d bytes, %d accumulator rows per panel, pieces of %d, "
                "%d row(s) cut across panels, %.1f %% padding, %.0f MB"
                % (i.sweep_panels, i.sweep_tiles, 16 * i.sweep_lanes, i.sweep_acc_rows, i.sweep_piece, i.sweep_split_rows,
                   100.0 * (i.sweep_slots - w.nnz) / max(w.nnz, 1), i.device_bytes / 1e6))
    if i.rowblock_steps > 0:
        return ("row-block plan: %d blocks, %d steps x %d table rows%s, %.1f %% of the nonzeros from LDS, %.0f MB"
                % (i.rowblock_blocks, i.rowblock_steps, i.rowblock_table_rows,
                   " (a table of consecutive columns per block)" if i.rowblock_local_tables else "",
                   100.0 * i.hot_nnz / max(w.nnz, 1), i.device_bytes / 1e6))
    text = "plan: %d column slab(s) of %d, sliced, %.0f MB" % (i.num_slabs, i.slab_cols, i.device_bytes / 1e6)
    if i.resident_cols:
        text += ", streaming hint on gathers outside the %d busiest columns (%.1f %% of the nonzeros)" % (
            i.resident_cols, 100.0 * (1.0 - i.resident_nnz / max(w.nnz, 1)))
    if i.hot_rows:
        text += ", %d hot columns per slab in LDS (%.1f %% of the nonzeros)" % (i.hot_rows, 100.0 * i.hot_nnz / max(w.nnz, 1))
    return text


def kernels_of(info, cus):
    """Which kernel each phase of a product launches for this kind of plan (None: the phase launches nothing)."""
    if info is None:
        return {"PREPARE": None, "MAIN": "mp_spmm_kernel", "FIXUP": "mp_fixup_kernel", "REDUCE": None}
    if info.sweep_panels > 0:
        return {"PREPARE": None, "MAIN": "sw_spmm_kernel", "FIXUP": "sw_fixup_kernel" if info.sweep_split_rows > 0 else None,
                "REDUCE": None}
    if info.rowblock_steps > 0:
        # a plan of one step and one round of blocks, or with local tables, reads its tables from X in the main kernel
        from_x = info.rowblock_local_tables or (info.rowblock_steps == 1 and info.rowblock_blocks <= cus)
        return {"PREPARE": None if from_x else "rb_gather_hot_kernel", "MAIN": "rb_spmm_kernel", "FIXUP": None, "REDUCE": None}
    return {"PREPARE": None, "MAIN": "mp_spmm_kernel (hot + cold launch)" if info.hot_rows > 0 else "mp_spmm_kernel",
            "FIXUP": "mp_fixup_kernel", "REDUCE": "tile_reduce_kernel" if info.num_slabs > 1 else None}


def phase_times(torch, PH, step, kernels, steps):
    """Average duration of every phase that launches something, from HIP events on the launch stream, over `steps`
    products phase by phase; None for a phase that launches nothing."""
    order = [("PREPARE", PH.MPS_PHASE_PREPARE), ("MAIN", PH.MPS_PHASE_MAIN), ("FIXUP", PH.MPS_PHASE_FIXUP),
             ("REDUCE", PH.MPS_PHASE_REDUCE)]
    live = [(name, ph) for name, ph in order if kernels[name] is not None]
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(len(live) + 1)] for _ in range(steps)]
    torch.cuda.synchronize()
    for row in evs:
        row[0].record()
        for k, (_, ph) in enumerate(live):
            step(ph)
            row[k + 1].record()
    torch.cuda.synchronize()
    out = {kernels[name]: None for name, _ in order if kernels[name] is not None}
    for k, (name, _) in enumerate(live):
        out[kernels[name]] = round(sum(r[k].elapsed_time(r[k + 1]) for r in evs) / steps, 5)
    return out


GATE_F32 = "|err| <= 1e-5 * sum_j |a_ij x_jk| + 1e-6 per element and ||err|| / ||ref|| <= 1e-5 against the fp64 row loop"
GATE_F16 = "|err| <= 2e-2 * |ref| + 2e-5 * sum_j |a_ij x_jk| + 1e-6 per element and ||err|| / ||ref|| <= 2e-2 against the fp64 row loop"


def check_product(np, orc, w, Yg, with_cpu_loop=None):
    """The product against the oracle's fp64 row loop: the gate the tests pin (relative to sum_j |a_ij x_jk| where rows
    are long and their terms cancel), and beside it how many elements miss the bar read literally."""
    ref, scale = (orc.spmm_f64_f16in if w.f16 else orc.spmm_f64)(w.rp, w.ci, w.val, w.X, want_abs=True)
    Yg = Yg.astype(np.float64)
    err_g = np.abs(Yg - ref)
    literal = (2e-2 * np.abs(ref) + 1e-6) if w.f16 else (1e-5 * np.abs(ref) + 1e-6)
    gate = (2e-2 * np.abs(ref) + 2e-5 * scale + 1e-6) if w.f16 else (1e-5 * scale + 1e-6)
    rel_fro = float(np.linalg.norm(err_g) / max(np.linalg.norm(ref), 1e-30))
    ok = bool(np.isfinite(Yg).all() and rel_fro <= (2e-2 if w.f16 else 1e-5) and (err_g <= gate).all())
    out = {"ok": ok, "gate": GATE_F16 if w.f16 else GATE_F32, "rel_fro": rel_fro, "max_abs_err": float(err_g.max()),
           "elements": int(ref.size), "outside_literal_bar_gpu": int((err_g > literal).sum()),
           "literal_bar": "|err| <= 2e-2 |ref| + 1e-6 (fp16)" if w.f16 else "|err| <= 1e-5 |ref| + 1e-6"}
    if with_cpu_loop is not None:
        out["outside_literal_bar_cpu_fp32_loop"] = int((np.abs(with_cpu_loop.astype(np.float64) - ref) > literal).sum())
    return out


def describe_plan(name, w, plan, g, tpw_arg, cost):
    """The config fields that say what ran: cost, partitions and partitions per wavefront only for plans that have them."""
    info = plan.info if plan is not None else None
    slab = info is None or (info.sweep_panels == 0 and info.rowblock_steps == 0)
    return {"layout": layout_text(w, plan), "plan_signature": plan_signature(name, info),
            "cost": cost if slab else None, "partitions": (info.num_partitions if info is not None else None) if slab else None,
            "threads_per_wave": (tpw_arg or g.max_threads_per_wave(w.K, w.eb)) if slab else None,
            "plan_bytes": int(info.device_bytes) if info is not None else 0,
            "plan_built_on": None if info is None else ("device" if info.built_on_device else "host"),
            "csr_bytes": int(4 * (w.n + 1) + (4 + w.eb) * w.nnz)}


def calibrate_copy(torch, dev):
    """A plain device copy of known size, for scaling the FETCH_SIZE / WRITE_SIZE counters:
    rocprofv3 --pmc FETCH_SIZE -- python3 bench.py --calibrate-copy   (then the same with WRITE_SIZE)."""
    n = 1 << 28  # 1 GiB of fp32 read, 1 GiB written
    a = torch.ones(n, dtype=torch.float32, device=dev)
    b = torch.empty_like(a)
    for _ in range(5):
        b.copy_(a)
    torch.cuda.synchronize()
    print(json.dumps({"calibrate_copy": {"bytes_read_per_copy": 4 * n, "bytes_written_per_copy": 4 * n, "copies": 5,
                                         "kernel": "the elementwise copy kernel torch launches for Tensor.copy_"}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=100,
                    help="untimed steps first: the first ~70 products after an idle GPU run about 4 %% slower than the rest")
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
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
    ap.add_argument("--sweep", default="auto", choices=["auto", "off", "force"],
                    help="sweep plan (rows summed in LDS, nonzeros visited in column order): where the library picks it / "
                         "never / always")
    ap.add_argument("--sweep-piece", type=int, default=0, help="sweep plans: most entries of a row per accumulator row (0 = library default)")
    ap.add_argument("--sweep-together", type=int, default=0, help="sweep plans: 1 or 2 instructions added up at the same time (0 = library default)")
    ap.add_argument("--sweep-acc-rows", type=int, default=0, help="sweep plans: most accumulator rows per panel (0 = what fits in LDS)")
    ap.add_argument("--rb-steps", type=int, default=0, help="steps (LDS tables) of a row-block plan (0 = library default)")
    ap.add_argument("--rb-table-rows", type=int, default=0, help="rows per LDS table of a row-block plan (0 = what fits)")
    ap.add_argument("--resident", default="auto", choices=["auto", "off"],
                    help="untiled plans: streaming hint on the gathers of unpopular columns where the library picks it / never")
    ap.add_argument("--column-tiles", default="auto", choices=["auto", "off"],
                    help="untiled plans with rows of X of 512 bytes and more: passes over 128-byte column tiles where the "
                         "library picks them / never")
    ap.add_argument("--resident-bytes", type=int, default=0, help="rows of X gathered without the hint (0 = library default)")
    ap.add_argument("--values", default="uniform", choices=["uniform", "degree", "gcn"],
                    help="edge values: U[0,1), or the reference's deg(r) * deg(c), or 1 / sqrt(deg(r) * deg(c)), as a value array")
    ap.add_argument("--weights", default="none", choices=["none", "degree", "gcn"],
                    help="plan with degree weights: the same weights formed from one factor per node, no value array "
                         "(fp32; the check then compares with the value array of the same weights)")
    ap.add_argument("--slab-bytes", type=int, default=0, help="slab size for tiling (0 = library default)")
    ap.add_argument("--tpw", type=int, default=0, help="partitions per wavefront (0 = full wavefront)")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--graph", action="store_true",
                    help="capture one step in a HIP graph and time replays (what a launch-bound caller would do)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and the result check")
    ap.add_argument("--no-configs", action="store_true", help="time the one workload only, not the other configurations")
    ap.add_argument("--calibrate-copy", action="store_true", help="run a plain 1 GiB device copy five times and exit (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported (no multi-GPU path exists)" % args.gpus)

    import numpy as np
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        calibrate_copy(torch, dev)
        return
    pkg = entry.load_package()
    sp, g = pkg.spmm, pkg.graphs
    PH = pkg._cabi
    spec, K, dt = WORKLOADS[args.workload]
    custom = False
    if args.spec:
        spec, custom = args.spec, True
    if args.k:
        K, custom = args.k, True
    if args.dtype:
        dt, custom = args.dtype, True
    name = "custom" if custom else args.workload
    if args.weights != "none":
        args.values, custom = args.weights, True
    elif args.values != "uniform":
        custom = True
    name = "custom" if custom else args.workload
    w = Workload(pkg, name, spec, K, dt, args.seed, torch, dev, values=args.values)
    if args.weights != "none":
        # no value per nonzero is read; two factors per node are
        w.b_alg = algorithmic_bytes(w.n, w.nnz, K, 0, w.eb) + 8 * w.n

    def make_plan(wl, **overrides):
        cost = args.cost if args.cost > 0 else sp.default_cost(wl.n, wl.nnz, wl.K, wl.eb)
        kw = dict(cost=cost, threads_per_wave=args.tpw, tiling={"auto": "auto", "untiled": "off", "tiled": "force", "plain": "auto"}[args.mode],
                  slab_bytes=args.slab_bytes, hot=args.hot, rowblock=args.rowblock, rowblock_steps=args.rb_steps,
                  rowblock_table_rows=args.rb_table_rows, keep_sources=False, resident=args.resident,
                  resident_bytes=args.resident_bytes, weights=None if args.weights == "none" else args.weights,
                  column_tiles=args.column_tiles == "auto", sweep=args.sweep, sweep_piece=args.sweep_piece,
                  sweep_acc_rows=args.sweep_acc_rows, sweep_together=args.sweep_together)
        kw.update(overrides)
        return sp.Plan(wl.csr, wl.K, **kw), cost

    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    orc = None if args.no_cpu else entry.load_oracle()

    def prepare(wl, plain=False, **overrides):
        """The per-matrix preprocessing for one kind of plan, and how long it takes (a second plan of the same kind,
        built and timed before any product and before the check against the CPU loops, whose OpenMP threads keep
        spinning for a while after their loop and would share the cores with the builder's)."""
        plan, sched = None, None
        cost = args.cost if args.cost > 0 else sp.default_cost(wl.n, wl.nnz, wl.K, wl.eb)
        if plain:
            sched = sp.generate_mp_sched(wl.csr.row_ptr, wl.nnz, cost=cost)
        else:
            plan, cost = make_plan(wl, **overrides)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        if plan is not None:
            make_plan(wl, **overrides)[0].close()
        else:
            sp.generate_mp_sched(wl.csr.row_ptr, wl.nnz, cost=cost)
        torch.cuda.synchronize()
        return plan, sched, cost, round((time.perf_counter() - t1) * 1e3, 3)

    def measure(wl, wname, prepared, steps, warmup, graph=False, cpu_loop=None, defer_check=False, busy_ms=0.0):
        """One workload with one prepared plan: exactly `steps` timed products after `warmup` untimed ones, then the
        per-kernel durations, the counter readings on file for that plan shape, and the check against the fp64 row
        loop.  busy_ms: the untimed products go on, ten at a time, until the device has worked that long - a GPU that
        idled for some tens of milliseconds needs about 30 ms of work before its clocks are back up."""
        plan, sched, cost, preprocessing_ms = prepared
        info = plan.info if plan is not None else None

        def step(phases=None):
            if plan is not None:
                plan.spmm(wl.d_X, out=wl.d_Y, phases=phases)
            else:
                sp.spmm_merge_path(wl.csr, wl.d_X, sched, threads_per_wave=args.tpw, out=wl.d_Y, phases=phases)

        warmed = 0
        t_busy = time.perf_counter()
        while warmed < warmup or (time.perf_counter() - t_busy) * 1e3 < busy_ms:
            for _ in range(min(10, warmup - warmed) if warmed < warmup else 10):
                step()
                warmed += 1
            if busy_ms > 0.0:
                torch.cuda.synchronize()
        timed_step = step
        if graph:
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
        # ---- timed region: exactly `steps` steps, inputs already in HBM ----------
        ms, wall_ms = time_steps(torch, timed_step, steps, warmup if graph else 0)
        kernels = kernels_of(info, cus)
        kernel_ms = phase_times(torch, PH, step, kernels, steps)
        main_name = kernels["MAIN"]
        main_ms = kernel_ms[main_name]
        desc = describe_plan(wname, wl, plan, g, args.tpw, cost)
        if plan is None:
            desc["partitions"] = sched.P
        traffic, l2_hit, where, gather_hit = measured_counters(desc["plan_signature"], with_requests=True,
                                                               other_lines=lines_read_once(wl, info))
        res = {"ms_per_step": round(ms, 5), "wall_ms_per_step": round(wall_ms, 5), "gflops": round(wl.flops / (ms * 1e6), 2),
               "steps": steps, "warmup": warmed,
               "kernel_ms": kernel_ms, "main_kernel": main_name,
               "phases": {k.lower(): v for k, v in kernels.items()},  # the kernel each phase launches; null: nothing
               "frac_step": round(wl.b_alg / (ms * 1e6) / PEAK_HBM_GBS, 4),
               "frac_main_kernel": round(wl.b_alg / (main_ms * 1e6) / PEAK_HBM_GBS, 4),
               "traffic": traffic, "l2_hit_rate": l2_hit, "l2_hit_rate_gathers_est": gather_hit, "counters_from": where,
               "algorithmic_bytes": int(wl.b_alg)}
        res.update(desc)
        res["preprocessing_ms"] = preprocessing_ms
        if orc is not None:
            if defer_check:
                res["_Y"] = wl.d_Y.clone()  # the caller checks it later; the device is not kept waiting for a copy to the host
            else:
                res["check"] = check_product(np, orc, wl, wl.d_Y.float().cpu().numpy(), cpu_loop)
        if plan is not None:
            plan.close()
        return res

    def run(wl, wname, steps, warmup, plain=False, **kw):
        overrides = {k: kw.pop(k) for k in list(kw) if k not in ("graph", "cpu_loop", "defer_check", "busy_ms")}
        return measure(wl, wname, prepare(wl, plain=plain, **overrides), steps, warmup, **kw)

    with_configs = not args.no_configs and not custom and args.workload == HEADLINE
    steps_c, warm_c = min(args.steps, 30), min(args.warmup, 10)
    kBusyMs = 40.0  # configurations beside the headline: untimed products for at least this long
    # The GPU's run first: the CPU baseline below keeps the host busy for ten seconds, during which an idle GPU drops
    # its clocks, and the products that follow would be timed while they come back up.
    # And of the two plans of the headline matrix the merge-path slab plan first (partitioner, LDS-staged windows,
    # carry-out fix-up: a `configs` entry), the library's own plan straight after it: both are prepared before either is
    # timed, so that the headline's `--warmup` products find a device that is already at work, as every later product
    # of a caller's loop does.
    head_prepared = prepare(w, plain=args.mode == "plain")
    slab_row = None
    if with_configs:
        r = measure(w, name, prepare(w, rowblock="off", sweep="off"), steps_c, warm_c, defer_check=True, busy_ms=kBusyMs)
        slab_row = dict({"workload": name + "|slab", "n_rows": int(w.n), "nnz": int(w.nnz), "K": K, "dtype": dt}, **r)
    head = measure(w, name, head_prepared, args.steps, args.warmup, graph=args.graph, defer_check=True)
    cpu = None
    Yc = None
    if orc is not None:
        # CPU baseline leg: the oracle's multithreaded fp32 CSR x dense loop on this box's host cores,
        # bounded to a few passes over the same workload.
        present = os.cpu_count() or 1
        threads = max(1, min(present, orc.max_threads()))
        val32 = w.val.astype(np.float32) if w.f16 else w.val
        X32 = w.X.astype(np.float32) if w.f16 else w.X
        Yc = np.empty((w.n, K), dtype=np.float32)
        orc.spmm_f32_mt(w.rp, w.ci, val32, X32, threads=threads, out=Yc)  # warm
        passes, spent = 0, 0.0
        while passes < 1000 and spent < 10.0:  # about 10 s of CPU work
            c0 = time.perf_counter()
            orc.spmm_f32_mt(w.rp, w.ci, val32, X32, threads=threads, out=Yc)
            spent += time.perf_counter() - c0
            passes += 1
        cpu_s = spent / passes
        cpu = {"value": round(w.flops / cpu_s / 1e9, 3), "unit": "GFLOP/s", "cores": threads, "cores_present": present,
               "kind": "port", "sample": "%d full passes over the same workload, %.3f s each" % (passes, cpu_s)}

    if orc is not None:
        head["check"] = check_product(np, orc, w, head.pop("_Y").float().cpu().numpy(), Yc)
        if slab_row is not None:
            slab_row["check"] = check_product(np, orc, w, slab_row.pop("_Y").float().cpu().numpy(), None)
    achieved = w.b_alg / (head["kernel_ms"][head["main_kernel"]] * 1e6)
    out = {
        "metric": "SpMM GFLOP/s (2*nnz*K/t), merge-path CSR x row-major dense",
        "value": head["gflops"],
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "scaling_note": "one GPU only: nothing is scaled",
        "vs_baseline": None,
        "dtype": dt,
        "data": "synthetic (seeded generator, values U[0,1), features U[-1,1))",
        "launch": "one HIP graph replay per step" if args.graph else "kernel launches per step",
        "config": {"workload": name, "spec": spec, "n_rows": int(w.n), "nnz": int(w.nnz), "K": K,
                   "max_row_degree": int(w.max_deg), "cost": head["cost"], "partitions": head["partitions"],
                   "threads_per_wave": head["threads_per_wave"], "seed": args.seed,
                   "values": args.values, "weights": "value array" if args.weights == "none" else "one factor per node (no value array)",
                   "layout": head["layout"], "plan_signature": head["plan_signature"],
                   "plan_bytes": head["plan_bytes"], "plan_built_on": head["plan_built_on"], "csr_bytes": head["csr_bytes"]},
        "gbs_algorithmic_per_step": round(w.b_alg / (head["ms_per_step"] * 1e6), 2),
        "hbm_fraction_per_step": head["frac_step"],
        "kernel_ms": dict(head["kernel_ms"], **{"preprocessing, host wall time (once per matrix)": head["preprocessing_ms"]}),
        "phases": head["phases"],
        "wall_ms_per_step": head["wall_ms_per_step"],
        "roofline": {"bound": "hbm", "kernel": head["main_kernel"], "achieved": round(achieved, 2), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 4), "traffic": head["traffic"],
                     "l2_hit_rate": head["l2_hit_rate"], "l2_hit_rate_gathers_est": head["l2_hit_rate_gathers_est"],
                     "traffic_from": head["counters_from"],
                     "algorithmic_bytes": int(w.b_alg)},
        "host_generate_s": round(w.gen_s, 2),
    }
    ok = True
    if cpu is not None:
        out["cpu_baseline"] = cpu
        out["check_vs_cpu_fp32"] = head["check"]
        ok = head["check"]["ok"]

    if with_configs:
        # the other configurations of the benchmark, each with the library's own plan and the same timed loop, after
        # the headline graph's slab plan from above
        rows = [slab_row]
        del w
        torch.cuda.empty_cache()
        for cname in OTHER_CONFIGS:
            cspec, cK, cdt = WORKLOADS[cname]
            wl = Workload(pkg, cname, cspec, cK, cdt, args.seed, torch, dev)
            r = run(wl, cname, steps_c, warm_c, busy_ms=kBusyMs)
            rows.append(dict({"workload": cname, "n_rows": int(wl.n), "nnz": int(wl.nnz), "K": cK, "dtype": cdt}, **r))
            del wl
            torch.cuda.empty_cache()
        for r in rows:
            r["frac"] = r["frac_step"]
            if "check" in r:
                ok = ok and r["check"]["ok"]
        out["configs"] = rows
        out["configs_note"] = ("frac = algorithmic bytes / whole-step time / 8 TB/s, frac_main_kernel the same over the main "
                               "kernel's time; %d steps each, after at least %d untimed ones and %d ms of them (`warmup` per entry: a GPU "
                               "that idled needs about 30 ms of work before its clocks are back up); the slab plan of the "
                               "headline matrix is timed before the headline's own warm-up; kernel_ms: a phase that "
                               "launches nothing has no entry; traffic and l2_hit_rate from the counter runs under profiles/"
                               % (steps_c, warm_c, int(kBusyMs)))

    print(json.dumps(out))
    if not ok:
        sys.exit("bench.py: a product is outside the tolerance of the fp64 row loop")


if __name__ == "__main__":
    main()
