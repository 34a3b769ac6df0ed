// rocsparse_spmm_row / rocsparse_spmm_col <input_file> <DIM> <repeat> [--alg default|row_split|merge_path|nnz_split]
// Vendor-library comparison drivers: the MI355X counterpart of
// src/cusparse_spmm_row.cu and src/cusparse_spmm_col.cu (same command line,
// :36-38; same generic-API call sequence, :165-202), with rocSPARSE's
// rocsparse_spmm in place of cusparseSpMM.  Dense matrices are row-major
// (ld = DIM) or, with -DMPS_COL_MAJOR, column-major (ld = N), as at :172-176
// of the two reference programs.  Unlike the reference, the timed loop is
// bracketed by device events (the reference times the launches without a
// device synchronisation, :193-208).
#include <rocsparse/rocsparse.h>

#include "driver_common.hpp"

#define RS_OK(expr)                                                                             \
    do {                                                                                        \
        rocsparse_status s_ = (expr);                                                           \
        if (s_ != rocsparse_status_success) drv::die(std::string(#expr) + ": rocsparse status " + std::to_string((int)s_)); \
    } while (0)

int main(int argc, char **argv)
{
    using namespace drv;
    Options opt;
    std::string alg_name = "default";
    std::vector<std::string> raw(argv, argv + argc), keep{raw[0]};
    for (size_t i = 1; i < raw.size(); ++i) {
        if (raw[i] == "--alg" && i + 1 < raw.size()) alg_name = raw[++i];
        else keep.push_back(raw[i]);
    }
    std::vector<char *> kargv;
    for (auto &s : keep) kargv.push_back(const_cast<char *>(s.c_str()));
    std::vector<std::string> pos = split_args((int)kargv.size(), kargv.data(), opt);
    if (pos.size() < 3) {
        std::cout << "Usage: ./application <input_file> <DIM> <repeat>" << std::endl;
        std::exit(-1);
    }
    const int K = std::atoi(pos[1].c_str());
    const int repeats = std::atoi(pos[2].c_str());
    if (K < 1) die("DIM must be positive");
    rocsparse_spmm_alg alg = rocsparse_spmm_alg_default;
    if (alg_name == "row_split") alg = rocsparse_spmm_alg_csr_row_split;
    else if (alg_name == "merge_path") alg = rocsparse_spmm_alg_csr_merge_path;
    else if (alg_name == "nnz_split") alg = rocsparse_spmm_alg_csr_nnz_split;
    else if (alg_name != "default") die("unknown --alg " + alg_name);
#ifdef MPS_COL_MAJOR
    const bool col_major = true;
#else
    const bool col_major = false;
#endif

    Graph gr;
    load_graph(pos[0], opt.seed, gr);
    const int N = gr.n_rows, nnz = gr.nnz;
    std::vector<float> h_val((size_t)nnz), h_X((size_t)N * K), h_Y((size_t)N * K), h_in((size_t)N * K);
    mps_ok(mps_fill_uniform_f32(h_val.data(), h_val.size(), kSeedVal, 0.0f, 1.0f), "fill val");
    mps_ok(mps_fill_uniform_f32(h_X.data(), h_X.size(), kSeedX, -1.0f, 1.0f), "fill X");
    if (col_major) {
        for (int i = 0; i < N; ++i)
            for (int k = 0; k < K; ++k) h_in[(size_t)k * N + i] = h_X[(size_t)i * K + k];
    } else {
        h_in = h_X;
    }
    DevBuf<int> d_rp((size_t)N + 1), d_ci((size_t)nnz);
    DevBuf<float> d_val((size_t)nnz), d_X((size_t)N * K), d_Y((size_t)N * K);
    d_rp.upload(mps_graph_row_ptr(gr.g));
    d_ci.upload(mps_graph_col_idx(gr.g));
    d_val.upload(h_val.data());
    d_X.upload(h_in.data());

    rocsparse_handle handle;
    rocsparse_spmat_descr matA;
    rocsparse_dnmat_descr matB, matC;
    RS_OK(rocsparse_create_handle(&handle));
    RS_OK(rocsparse_create_csr_descr(&matA, N, N, nnz, d_rp.p, d_ci.p, d_val.p, rocsparse_indextype_i32,
                                     rocsparse_indextype_i32, rocsparse_index_base_zero, rocsparse_datatype_f32_r));
    const rocsparse_order order = col_major ? rocsparse_order_column : rocsparse_order_row;
    const int64_t ld = col_major ? N : K;
    RS_OK(rocsparse_create_dnmat_descr(&matB, N, K, ld, d_X.p, rocsparse_datatype_f32_r, order));
    RS_OK(rocsparse_create_dnmat_descr(&matC, N, K, ld, d_Y.p, rocsparse_datatype_f32_r, order));
    const float alpha = 1.0f, beta = 0.0f;
    size_t buffer_size = 0;
    RS_OK(rocsparse_spmm(handle, rocsparse_operation_none, rocsparse_operation_none, &alpha, matA, matB, &beta, matC,
                         rocsparse_datatype_f32_r, alg, rocsparse_spmm_stage_buffer_size, &buffer_size, nullptr));
    DevBuf<unsigned char> d_buf(buffer_size);
    Timing prep = time_launches(0, 1, [&] {
        RS_OK(rocsparse_spmm(handle, rocsparse_operation_none, rocsparse_operation_none, &alpha, matA, matB, &beta, matC,
                             rocsparse_datatype_f32_r, alg, rocsparse_spmm_stage_preprocess, &buffer_size, d_buf.p));
    });
    hip_ok(hipMemset(d_Y.p, 0xff, d_Y.n * sizeof(float)), "hipMemset");
    Timing t = time_launches(opt.warmup, repeats, [&] {
        RS_OK(rocsparse_spmm(handle, rocsparse_operation_none, rocsparse_operation_none, &alpha, matA, matB, &beta, matC,
                             rocsparse_datatype_f32_r, alg, rocsparse_spmm_stage_compute, &buffer_size, d_buf.p));
    });
    d_Y.download(h_in.data());
    if (col_major) {
        for (int i = 0; i < N; ++i)
            for (int k = 0; k < K; ++k) h_Y[(size_t)i * K + k] = h_in[(size_t)k * N + i];
    } else {
        h_Y = h_in;
    }
    double checksum = finish_output(h_Y, N, K, opt);  // --dump always writes row-major
    std::printf("rocsparse_spmm alg %s, %s-major dense, workspace %zu B, preprocess %.2f us\n", alg_name.c_str(),
                col_major ? "column" : "row", buffer_size, prep.avg_us);
    char extra[160];
    std::snprintf(extra, sizeof extra, ", \"alg\": \"%s\", \"order\": \"%s\", \"preprocess_us\": %.3f", alg_name.c_str(),
                  col_major ? "col" : "row", prep.avg_us);
    report(col_major ? "rocsparse_spmm_col" : "rocsparse_spmm_row", "fp32", N, nnz, K, 4, 4, repeats, t, checksum, extra);
    rocsparse_destroy_spmat_descr(matA);
    rocsparse_destroy_dnmat_descr(matB);
    rocsparse_destroy_dnmat_descr(matC);
    rocsparse_destroy_handle(handle);
    return 0;
}
