// main() of MergePathSpMM and MergePathSpMM_fp16, templated on the element
// type.  Command line of src/MergePathSpMM.cu:114-124:
//   <input_file> <dimension> <cost> <threads_per_wave> <repeat>
#ifndef MPS_MERGEPATH_DRIVER_HPP
#define MPS_MERGEPATH_DRIVER_HPP

#include "driver_common.hpp"

namespace drv {

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr const char *name = "fp32";
    static int fill(float *p, size_t n, uint64_t seed, float lo, float hi) { return mps_fill_uniform_f32(p, n, seed, lo, hi); }
    static int spmm(const int *rp, const int *ci, const float *v, const float *X, float *Y, int n, int nnz, int K, int P,
                    const int *cx, const int *cy, int tpw, void *ws, size_t wsb)
    { return mps_spmm_f32(rp, ci, v, X, Y, n, nnz, K, P, cx, cy, tpw, ws, wsb, nullptr); }
    static int plan_spmm(const mps_plan *pl, const float *X, float *Y) { return mps_plan_spmm_f32(pl, X, Y, nullptr); }
    static int degree_values(const int *rp, const int *ci, int n, int nnz, int mode, float *v)
    { return mps_degree_values_f32(rp, ci, n, nnz, mode, v, nullptr); }
    static float one() { return 1.0f; }
};
template <> struct Elem<uint16_t> {
    static constexpr const char *name = "fp16";
    static int fill(uint16_t *p, size_t n, uint64_t seed, float lo, float hi) { return mps_fill_uniform_f16(p, n, seed, lo, hi); }
    static int spmm(const int *rp, const int *ci, const uint16_t *v, const uint16_t *X, uint16_t *Y, int n, int nnz, int K,
                    int P, const int *cx, const int *cy, int tpw, void *ws, size_t wsb)
    { return mps_spmm_f16(rp, ci, v, X, Y, n, nnz, K, P, cx, cy, tpw, ws, wsb, nullptr); }
    static int plan_spmm(const mps_plan *pl, const uint16_t *X, uint16_t *Y) { return mps_plan_spmm_f16(pl, X, Y, nullptr); }
    static int degree_values(const int *rp, const int *ci, int n, int nnz, int mode, uint16_t *v)
    { return mps_degree_values_f16(rp, ci, n, nnz, mode, v, nullptr); }
    static uint16_t one() { return 0x3c00; }  // 1.0 in IEEE half
};

template <typename T>
int mergepath_main(int argc, char **argv)
{
    Options opt;
    std::vector<std::string> pos = split_args(argc, argv, opt);
    if (pos.size() < 5) {
        std::cout << "Usage: ./application <input_file> <dimension> <cost> <threads_per_wave> <repeat>" << std::endl;
        std::exit(-1);
    }
    const int dimension = std::atoi(pos[1].c_str());
    const bool tune = pos[2] == "auto";  // sweep cost / partitions per wavefront on this matrix first
    int cost = tune ? 0 : parse_cost(pos[2]);
    int threads_per_wave = std::atoi(pos[3].c_str());
    const int repeats = std::atoi(pos[4].c_str());
    if (dimension < 1) die("dimension must be positive");
    if (cost < 0) die("cost must be positive");

    Graph gr;
    load_graph(pos[0], opt.seed, gr);
    const int N = gr.n_rows, nnz = gr.nnz, K = dimension;
    if (cost == 0) mps_ok(mps_default_cost(N, nnz, K, (int)sizeof(T), &cost), "mps_default_cost");

    int max_tpw = 0;
    mps_ok(mps_max_threads_per_wave(K, (int)sizeof(T), &max_tpw), "mps_max_threads_per_wave");
    // "64" (or 0) asks for a full wavefront; otherwise the bound of src/MergePathSpMM.cu:224-228
    if (threads_per_wave == 0 || threads_per_wave == 64) threads_per_wave = max_tpw;
    if (threads_per_wave < 1 || threads_per_wave > max_tpw) {
        std::cout << "Cannot process the given number of threads withing a warp." << std::endl;
        std::cout << "Max threads per warp can be " << max_tpw << std::endl;
        std::exit(-1);
    }

    int P = 0;
    mps_ok(mps_num_partitions(N, nnz, cost, &P), "mps_num_partitions");

    std::vector<T> h_val((size_t)nnz), h_X((size_t)N * K), h_Y((size_t)N * K);
    mps_ok(Elem<T>::fill(h_val.data(), h_val.size(), kSeedVal, 0.0f, 1.0f), "fill val");
    mps_ok(Elem<T>::fill(h_X.data(), h_X.size(), kSeedX, -1.0f, 1.0f), "fill X");
    if (opt.ones) std::fill(h_X.begin(), h_X.end(), Elem<T>::one());

    DevBuf<int> d_rp((size_t)N + 1), d_ci((size_t)nnz), d_cx((size_t)P + 1), d_cy((size_t)P + 1);
    DevBuf<T> d_val((size_t)nnz), d_X((size_t)N * K), d_Y((size_t)N * K);
    d_rp.upload(mps_graph_row_ptr(gr.g));
    d_ci.upload(mps_graph_col_idx(gr.g));
    d_val.upload(h_val.data());
    d_X.upload(h_X.data());
    mps_ok(mps_csr_validate(d_rp.p, d_ci.p, N, N, nnz, nullptr), "mps_csr_validate");
    // the reference's implicit weight deg(row) * deg(col) (:450,459), written out once
    if (opt.weights >= 0) {
        mps_ok(Elem<T>::degree_values(d_rp.p, d_ci.p, N, nnz, opt.weights, d_val.p), "mps_degree_values");
        if (opt.cpu) d_val.download(h_val.data());
    }
    if (opt.factors && (opt.weights < 0 || sizeof(T) != 4 || !opt.use_plan || tune))
        die("--factors needs --weights degree|gcn, fp32 and a plan");

    if (tune) {
        mps_tune_result best{}, tried[32];
        int n_tried = 32;
        mps_ok(mps_plan_autotune(d_rp.p, d_ci.p, d_val.p, N, nnz, K, (int)sizeof(T), d_X.p, d_Y.p, 5, nullptr, &best, tried,
                                 &n_tried), "mps_plan_autotune");
        for (int i = 0; i < n_tried && i < 32; ++i)
            std::printf("tune: cost %4d, threads_per_wave %2d, flags %2u, slab bytes %9llu: %9.2f us\n", tried[i].cost,
                        tried[i].threads_per_wave, tried[i].flags, tried[i].slab_bytes, tried[i].ms * 1e3);
        cost = best.cost;
        threads_per_wave = best.threads_per_wave;
        opt.tiling = (int)(best.flags & (MPS_PLAN_NO_TILING | MPS_PLAN_FORCE_TILING | MPS_PLAN_NO_ROWBLOCK | MPS_PLAN_FORCE_ROWBLOCK |
                                         MPS_PLAN_NO_SWEEP | MPS_PLAN_FORCE_SWEEP));
        opt.hot = (int)(best.flags & (MPS_PLAN_NO_HOT | MPS_PLAN_FORCE_HOT));
        opt.slab_bytes = (size_t)best.slab_bytes;
        opt.use_plan = true;
        mps_ok(mps_num_partitions(N, nnz, cost, &P), "mps_num_partitions");
    }

    // Everything that depends on the matrix alone is built once, outside the
    // repeat loop, as generate_mp_sched and its uploads are (:192-220): with a
    // plan (default) the tiled / sliced copy and the partition; with --no-plan
    // the partition of the caller's arrays only.
    size_t ws_bytes = 0;
    DevBuf<unsigned char> d_ws;
    mps_plan *plan = nullptr;
    mps_plan_info info{};
    Timing prep;
    hip_ok(hipMemset(d_Y.p, 0xff, d_Y.n * sizeof(T)), "hipMemset");
    Timing t;
    if (opt.use_plan) {
        hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize");
        mps_plan_options popt{};
        popt.flags = (unsigned)(opt.tiling | opt.hot) | MPS_PLAN_NO_SOURCES;  // the values never change here
        popt.slab_bytes = opt.slab_bytes;
        popt.degree_weights = opt.factors ? opt.weights + 1 : 0;
        prep = time_launches(0, 1, [&] {
            mps_ok(mps_plan_create_ex(d_rp.p, d_ci.p, opt.factors ? nullptr : d_val.p, N, nnz, K, (int)sizeof(T), cost,
                                      threads_per_wave, &popt, nullptr, &plan), "mps_plan_create_ex");
        });
        mps_ok(mps_plan_get_info(plan, &info), "mps_plan_get_info");
        P = info.num_partitions;
        t = time_launches(opt.warmup, repeats, [&] { mps_ok(Elem<T>::plan_spmm(plan, d_X.p, d_Y.p), "mps_plan_spmm"); });
    } else {
        mps_ok(mps_spmm_workspace_bytes(P, K, threads_per_wave, (int)sizeof(T), &ws_bytes), "mps_spmm_workspace_bytes");
        d_ws.alloc(ws_bytes);
        prep = time_launches(1, 3, [&] { mps_ok(mps_partition(d_rp.p, N, nnz, P, d_cx.p, d_cy.p, nullptr), "mps_partition"); });
        t = time_launches(opt.warmup, repeats, [&] {
            mps_ok(Elem<T>::spmm(d_rp.p, d_ci.p, d_val.p, d_X.p, d_Y.p, N, nnz, K, P, d_cx.p, d_cy.p, threads_per_wave, d_ws.p,
                                 ws_bytes), "mps_spmm");
        });
    }
    d_Y.download(h_Y.data());
    double checksum = finish_output(h_Y, N, K, opt);

    std::printf("partitions: %d (cost %d), threads_per_wave %d, max row degree %d\n", P, cost, threads_per_wave,
                gr.max_degree);
    if (plan && info.sweep_panels > 0)
        std::printf("plan: %d panels x %d column tile(s) of %d bytes, %d accumulator rows per panel, %lld entry slots for %d nonzeros, "
                    "%d row(s) cut across panels, %.1f MB of device memory\n",
                    info.sweep_panels, info.sweep_tiles, 16 * info.sweep_lanes, info.sweep_acc_rows, info.sweep_slots, nnz,
                    info.sweep_split_rows, info.device_bytes / 1e6);
    else if (plan && info.rowblock_steps > 0)
        std::printf("plan: %d row blocks, %d steps of %d table rows, %lld of %d nonzeros (%.1f %%) gathered from LDS, %.1f MB of device memory\n",
                    info.rowblock_blocks, info.rowblock_steps, info.rowblock_table_rows, info.hot_nnz, nnz,
                    nnz ? 100.0 * (double)info.hot_nnz / nnz : 0.0, info.device_bytes / 1e6);
    else if (plan)
        std::printf("plan: %d column slab(s) of %d columns, %lld sliced rounds, %.1f MB of device memory\n", info.num_slabs,
                    info.slab_cols, info.total_rounds, info.device_bytes / 1e6);
    if (plan && info.resident_cols > 0)
        std::printf("resident columns: %d (%.1f %% of the nonzeros); gathers of the other columns carry the streaming hint\n",
                    info.resident_cols, nnz ? 100.0 * (double)info.resident_nnz / nnz : 0.0);
    if (opt.factors) std::printf("degree weights: one factor per node, no value array\n");
    if (plan && info.hot_rows > 0)
        std::printf("hot columns: %d rows of X per slab in LDS, %lld of %d nonzeros (%.1f %%), %d of %d wavefronts\n",
                    info.hot_rows, info.hot_nnz, nnz, nnz ? 100.0 * (double)info.hot_nnz / nnz : 0.0, info.hot_waves,
                    info.num_waves);
    std::printf("preprocessing: %.2f us, once per matrix (not in the launch time below)\n", prep.avg_us);
    char extra[256];
    std::snprintf(extra, sizeof extra,
                  ", \"P\": %d, \"cost\": %d, \"threads_per_wave\": %d, \"plan\": %s, \"num_slabs\": %d, \"hot_rows\": %d, "
                  "\"rowblock_steps\": %d, \"sweep_panels\": %d, \"resident_cols\": %d, \"prep_us\": %.3f",
                  P, cost, threads_per_wave, plan ? "true" : "false", plan ? info.num_slabs : 1, plan ? info.hot_rows : 0,
                  plan ? info.rowblock_steps : 0, plan ? info.sweep_panels : 0, plan ? info.resident_cols : 0, prep.avg_us);
    mps_plan_destroy(plan);
    std::string more = extra;
    if (opt.cpu)
        more += cpu_baseline<T>(mps_graph_row_ptr(gr.g), mps_graph_col_idx(gr.g), h_val, h_X, h_Y, N, nnz, K, t.avg_us);
    report("merge_path", Elem<T>::name, N, nnz, K, opt.factors ? 0 : (int)sizeof(T), (int)sizeof(T), repeats, t, checksum, more);
    return 0;
}

}  // namespace drv
#endif
