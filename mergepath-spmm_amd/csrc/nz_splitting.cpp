// nz_splitting <input_file> <dimension> <part_size> <repeat>
// Nonzero-splitting comparison driver (counterpart of src/nz_splitting.cu's main(), :104-253).
#include "driver_common.hpp"

int main(int argc, char **argv)
{
    using namespace drv;
    Options opt;
    std::vector<std::string> pos = split_args(argc, argv, opt);
    if (pos.size() < 4) {
        std::cout << "Usage: ./application <input_file> <dimension> <part_size> <repeat>" << std::endl;
        std::exit(-1);
    }
    const int K = std::atoi(pos[1].c_str());
    const int part_size = std::atoi(pos[2].c_str());
    const int repeats = std::atoi(pos[3].c_str());
    if (K < 1 || part_size < 1) die("dimension and part_size must be positive");
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

    int max_parts = 0, num_parts = 0;
    mps_ok(mps_nzsplit_max_parts(N, nnz, part_size, &max_parts), "mps_nzsplit_max_parts");
    DevBuf<int> d_pp((size_t)max_parts + 1), d_pn((size_t)max_parts), d_scratch((size_t)N + 1 + 2048);
    mps_ok(mps_nzsplit_build(d_rp.p, N, part_size, d_pp.p, d_pn.p, max_parts, d_scratch.p, &num_parts, nullptr),
           "mps_nzsplit_build");
    Timing t = time_launches(opt.warmup, repeats, [&] {
        mps_ok(mps_nzsplit_spmm_f32(d_ci.p, d_val.p, d_X.p, d_Y.p, N, nnz, K, d_pp.p, d_pn.p, num_parts, nullptr),
               "mps_nzsplit_spmm_f32");
    });
    d_Y.download(h_Y.data());
    double checksum = finish_output(h_Y, N, K, opt);
    std::printf("neighbour groups: %d (part_size %d)\n", num_parts, part_size);
    char extra[128];
    std::snprintf(extra, sizeof extra, ", \"part_size\": %d, \"num_parts\": %d", part_size, num_parts);
    std::string more = extra;
    if (opt.cpu) more += cpu_baseline<float>(mps_graph_row_ptr(gr.g), mps_graph_col_idx(gr.g), h_val, h_X, h_Y, N, nnz, K, t.avg_us);
    report("nz_splitting", "fp32", N, nnz, K, 4, 4, repeats, t, checksum, more);
    return 0;
}
