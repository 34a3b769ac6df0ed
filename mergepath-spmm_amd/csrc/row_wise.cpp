// row_wise <input_file> <dimension> <num_warps> <repeat>
// Row-split comparison driver (counterpart of src/row_wise.cu's main(), :60-170).
// The reference prints the whole result matrix; here that is behind --print.
#include "driver_common.hpp"

int main(int argc, char **argv)
{
    using namespace drv;
    Options opt;
    std::vector<std::string> pos = split_args(argc, argv, opt);
    if (pos.size() < 4) {
        std::cout << "Usage: ./application <input_file> <dimension> <num_warps> <repeat>" << std::endl;
        std::exit(-1);
    }
    const int K = std::atoi(pos[1].c_str());
    const int num_warps = std::atoi(pos[2].c_str());
    const int repeats = std::atoi(pos[3].c_str());
    if (K < 1 || num_warps < 1) die("dimension and num_warps must be positive");
    Graph gr;
    load_graph(pos[0], opt.seed, gr);
    const int N = gr.n_rows, nnz = gr.nnz;

    std::vector<float> h_val((size_t)nnz), h_X((size_t)N * K), h_Y((size_t)N * K);
    mps_ok(mps_fill_uniform_f32(h_val.data(), h_val.size(), kSeedVal, 0.0f, 1.0f), "fill val");
    mps_ok(mps_fill_uniform_f32(h_X.data(), h_X.size(), kSeedX, -1.0f, 1.0f), "fill X");
    DevBuf<int> d_rp((size_t)N + 1), d_ci((size_t)nnz);
    DevBuf<float> d_val((size_t)nnz), d_X((size_t)N * K), d_Y((size_t)N * K);
    d_rp.upload(mps_graph_row_ptr(gr.g));
    d_ci.upload(mps_graph_col_idx(gr.g));
    d_val.upload(h_val.data());
    d_X.upload(h_X.data());
    mps_ok(mps_csr_validate(d_rp.p, d_ci.p, N, N, nnz, nullptr), "mps_csr_validate");
    hip_ok(hipMemset(d_Y.p, 0xff, d_Y.n * sizeof(float)), "hipMemset");
    Timing t = time_launches(opt.warmup, repeats, [&] {
        mps_ok(mps_rowwise_spmm_f32(d_rp.p, d_ci.p, d_val.p, d_X.p, d_Y.p, N, nnz, K, num_warps, nullptr), "mps_rowwise_spmm_f32");
    });
    d_Y.download(h_Y.data());
    double checksum = finish_output(h_Y, N, K, opt);
    char extra[128];
    std::snprintf(extra, sizeof extra, ", \"num_warps\": %d", num_warps);
    std::string more = extra;
    if (opt.cpu) more += cpu_baseline<float>(mps_graph_row_ptr(gr.g), mps_graph_col_idx(gr.g), h_val, h_X, h_Y, N, nnz, K, t.avg_us);
    report("row_wise", "fp32", N, nnz, K, 4, 4, repeats, t, checksum, more);
    return 0;
}
