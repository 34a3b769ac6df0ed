// Shared by the four driver programs: argument handling, graph loading,
// device buffers, event timing and the report.  The drivers keep the
// positional command lines of the reference programs and call the kernels
// only through the C ABI (mpspmm.h).
#ifndef MPS_DRIVER_COMMON_HPP
#define MPS_DRIVER_COMMON_HPP

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <string>
#include <thread>
#include <vector>

#include "mpspmm.h"

namespace drv {

constexpr double kPeakGBs = 8000.0;     // MI355X HBM3E
constexpr uint64_t kSeedVal = 11, kSeedX = 13, kSeedGraph = 1;

[[noreturn]] inline void die(const std::string &msg, int code = 1)
{
    std::cerr << "error: " << msg << std::endl;
    std::exit(code);
}

inline void hip_ok(hipError_t e, const char *what)
{
    if (e != hipSuccess) die(std::string(what) + ": " + hipGetErrorString(e));
}

inline void mps_ok(int status, const char *what)
{
    if (status != MPS_OK) {
        std::string m = std::string(what) + ": " + mps_status_string(status);
        if (status >= MPS_ERR_HIP) m += std::string(" (") + hipGetErrorString((hipError_t)(status - MPS_ERR_HIP)) + ")";
        die(m);
    }
}

struct Options {
    std::string dump_path;  // --dump FILE: raw little-endian result matrix
    bool print_matrix = false;  // --print: the "v-" text dump of src/row_wise.cu:162-168
    int warmup = 3;
    uint64_t seed = kSeedGraph;
    bool use_plan = true;       // --no-plan: CSR entry points on the caller's arrays, no preprocessing
    int tiling = 0;             // --tiling off|force (default: where it pays)
    size_t slab_bytes = 0;      // --slab-bytes N (default: the library's 3 MiB)
    int hot = 0;                // --hot off|force (default: where it pays)
    int weights = -1;           // --weights explicit|degree|gcn: seeded values (default), or from degrees on the device
    bool ones = false;          // --features ones: all features 1.0, as the reference sets them (src/MergePathSpMM.cu:180-182)
    bool cpu = false;           // --cpu: time the host row loop on the same inputs and compare the results
    bool factors = false;       // --factors (with --weights degree|gcn, fp32): a plan with degree weights, no value array
};

// Strips the optional trailing flags; returns the positional arguments.
inline std::vector<std::string> split_args(int argc, char **argv, Options &opt)
{
    std::vector<std::string> pos;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--dump" && i + 1 < argc) opt.dump_path = argv[++i];
        else if (a == "--print") opt.print_matrix = true;
        else if (a == "--cpu") opt.cpu = true;
        else if (a == "--factors") opt.factors = true;
        else if (a == "--no-plan") opt.use_plan = false;
        else if (a == "--slab-bytes" && i + 1 < argc) opt.slab_bytes = std::strtoull(argv[++i], nullptr, 10);
        else if (a == "--tiling" && i + 1 < argc) {
            std::string t = argv[++i];
            opt.tiling = t == "off" ? MPS_PLAN_NO_TILING : t == "force" ? MPS_PLAN_FORCE_TILING : 0;
        }
        else if (a == "--hot" && i + 1 < argc) {
            std::string t = argv[++i];
            opt.hot = t == "off" ? MPS_PLAN_NO_HOT : t == "force" ? MPS_PLAN_FORCE_HOT : 0;
        }
        else if (a == "--weights" && i + 1 < argc) {
            std::string t = argv[++i];
            opt.weights = t == "degree" ? MPS_WEIGHT_DEGREE_PRODUCT : t == "gcn" ? MPS_WEIGHT_GCN : -1;
        }
        else if (a == "--features" && i + 1 < argc) opt.ones = std::string(argv[++i]) == "ones";
        else if (a == "--warmup" && i + 1 < argc) opt.warmup = std::atoi(argv[++i]);
        else if (a == "--seed" && i + 1 < argc) opt.seed = std::strtoull(argv[++i], nullptr, 10);
        else pos.push_back(a);
    }
    return pos;
}

struct Graph {
    mps_graph *g = nullptr;
    int n_rows = 0, nnz = 0, max_degree = 0;
    ~Graph() { mps_graph_free(g); }
};

// <input_file> is a .csr text file, or "gen:<spec>" for a seeded synthetic graph.
inline void load_graph(const std::string &arg, uint64_t seed, Graph &out)
{
    if (arg.rfind("gen:", 0) == 0)
        mps_ok(mps_graph_generate(arg.c_str() + 4, seed, &out.g), "mps_graph_generate");
    else
        mps_ok(mps_graph_from_csr_file(arg.c_str(), &out.g), arg.c_str());
    mps_ok(mps_graph_dims(out.g, &out.n_rows, &out.nnz, &out.max_degree), "mps_graph_dims");
    // first output line of every reference program (src/MergePathSpMM.cu:141)
    std::cout << "Total number of rows: " << out.n_rows << " and non-zeros: " << out.nnz << std::endl;
}

template <typename T>
struct DevBuf {
    T *p = nullptr;
    size_t n = 0;
    DevBuf() = default;
    explicit DevBuf(size_t count) { alloc(count); }
    DevBuf(const DevBuf &) = delete;
    DevBuf &operator=(const DevBuf &) = delete;
    ~DevBuf() { if (p) (void)hipFree(p); }
    void alloc(size_t count)
    {
        n = count;
        hip_ok(hipMalloc(reinterpret_cast<void **>(&p), std::max<size_t>(count, 4) * sizeof(T)), "hipMalloc");
    }
    void upload(const T *h) { if (n) hip_ok(hipMemcpy(p, h, n * sizeof(T), hipMemcpyHostToDevice), "hipMemcpy H2D"); }
    void download(T *h) const { if (n) hip_ok(hipMemcpy(h, p, n * sizeof(T), hipMemcpyDeviceToHost), "hipMemcpy D2H"); }
};

struct Timing {
    double avg_us = 0, min_us = 0;
};

// Times `repeat` back-to-back calls of fn (one event pair around each) after warm-up.
template <typename F>
Timing time_launches(int warmup, int repeat, F &&fn)
{
    for (int i = 0; i < warmup; ++i) fn();
    hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize");
    Timing t;
    if (repeat < 1) return t;
    std::vector<hipEvent_t> ev(2 * (size_t)repeat);
    for (auto &e : ev) hip_ok(hipEventCreate(&e), "hipEventCreate");
    for (int i = 0; i < repeat; ++i) {
        hip_ok(hipEventRecord(ev[2 * i], nullptr), "hipEventRecord");
        fn();
        hip_ok(hipEventRecord(ev[2 * i + 1], nullptr), "hipEventRecord");
    }
    hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize");
    double sum = 0, mn = 1e30;
    for (int i = 0; i < repeat; ++i) {
        float ms = 0;
        hip_ok(hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]), "hipEventElapsedTime");
        sum += ms * 1e3;
        mn = std::min(mn, (double)ms * 1e3);
    }
    for (auto &e : ev) (void)hipEventDestroy(e);
    t.avg_us = sum / repeat;
    t.min_us = mn;
    return t;
}

// Algorithmic bytes of one SpMM: row_ptr + col_idx + val + dense in + dense out.
inline double algorithmic_bytes(int n_rows, int nnz, int K, int val_bytes, int elem_bytes)
{
    return 4.0 * (n_rows + 1.0) + 4.0 * nnz + (double)val_bytes * nnz + 2.0 * elem_bytes * (double)n_rows * K;
}

inline void report(const char *kernel, const char *dtype, int n_rows, int nnz, int K, int val_bytes,
                   int elem_bytes, int repeat, const Timing &t, double checksum, const std::string &extra_json)
{
    double flops = 2.0 * nnz * K;
    double bytes = algorithmic_bytes(n_rows, nnz, K, val_bytes, elem_bytes);
    double gflops = t.avg_us > 0 ? flops / (t.avg_us * 1e3) : 0;
    double gbs = t.avg_us > 0 ? bytes / (t.avg_us * 1e3) : 0;
    std::printf("kernel: %s (%s), K=%d, repeat=%d\n", kernel, dtype, K, repeat);
    std::printf("time per launch: avg %.2f us, min %.2f us\n", t.avg_us, t.min_us);
    std::printf("throughput: %.1f GFLOP/s (2*nnz*K/t), %.1f GB/s algorithmic = %.1f%% of %.0f GB/s\n", gflops, gbs,
                100.0 * gbs / kPeakGBs, kPeakGBs);
    std::printf("checksum: %.9e\n", checksum);
    std::printf("{\"kernel\": \"%s\", \"dtype\": \"%s\", \"n_rows\": %d, \"nnz\": %d, \"K\": %d, \"repeat\": %d, "
                "\"avg_us\": %.3f, \"min_us\": %.3f, \"gflops\": %.2f, \"gbs\": %.2f, \"roofline_frac\": %.4f, "
                "\"checksum\": %.9e%s}\n",
                kernel, dtype, n_rows, nnz, K, repeat, t.avg_us, t.min_us, gflops, gbs, gbs / kPeakGBs, checksum,
                extra_json.c_str());
}

inline float half_bits_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {
            int e = -1;
            do { ++e; man <<= 1; } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline double to_double(float v) { return v; }
inline double to_double(uint16_t v) { return half_bits_to_float(v); }

template <typename T>
double finish_output(const std::vector<T> &Y, int n_rows, int K, const Options &opt)
{
    double sum = 0;
    for (size_t i = 0; i < Y.size(); ++i) sum += to_double(Y[i]);
    if (!opt.dump_path.empty()) {
        FILE *f = std::fopen(opt.dump_path.c_str(), "wb");
        if (!f || std::fwrite(Y.data(), sizeof(T), Y.size(), f) != Y.size()) die("cannot write " + opt.dump_path);
        std::fclose(f);
    }
    if (opt.print_matrix) {
        // text layout of src/row_wise.cu:162-168
        for (int i = 0; i < n_rows; i++) {
            for (int j = 0; j < K; j++) std::cout << (float)to_double(Y[(size_t)i * K + j]) << "-";
            std::cout << std::endl;
        }
    }
    return sum;
}

// CPU baseline of the drivers (--cpu): the row loop the reference checks its kernels against
// (test/compare.h:18-31), in fp32 like the device (fp32 accumulation for half inputs too), rows dealt
// to the host threads in contiguous blocks of equal nonzero count.  Prints the time of one product,
// the threads used and present, and how far the device result is from it; returns the JSON fields.
template <typename T>
std::string cpu_baseline(const int *rp, const int *ci, const std::vector<T> &val, const std::vector<T> &X,
                         const std::vector<T> &Y_gpu, int n_rows, int nnz, int K, double gpu_us)
{
    const unsigned present = std::max(1u, std::thread::hardware_concurrency());
    // the host share of a one-GPU box is 16 cores; more threads than that only queue
    const unsigned threads = std::min(present, 16u);
    std::vector<float> Y((size_t)n_rows * K);
    std::vector<int> first(threads + 1, n_rows);
    first[0] = 0;
    for (unsigned t = 1; t < threads; ++t) {
        const long long want = (long long)nnz * t / threads;
        first[t] = (int)(std::lower_bound(rp, rp + n_rows + 1, (int)want) - rp);
        if (first[t] > n_rows) first[t] = n_rows;
    }
    auto pass = [&]() {
        std::vector<std::thread> pool;
        for (unsigned t = 0; t < threads; ++t)
            pool.emplace_back([&, t] {
                std::vector<float> acc((size_t)K);
                for (int r = first[t]; r < first[t + 1]; ++r) {
                    std::fill(acc.begin(), acc.end(), 0.f);
                    for (int e = rp[r]; e < rp[r + 1]; ++e) {
                        const float a = (float)to_double(val[(size_t)e]);
                        const T *x = X.data() + (size_t)ci[e] * K;
                        for (int k = 0; k < K; ++k) acc[(size_t)k] += a * (float)to_double(x[k]);
                    }
                    std::copy(acc.begin(), acc.end(), Y.begin() + (size_t)r * K);
                }
            });
        for (auto &th : pool) th.join();
    };
    pass();  // warm
    int passes = 0;
    double spent = 0;
    while (passes < 20 && spent < 5.0) {
        const auto t0 = std::chrono::steady_clock::now();
        pass();
        spent += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        ++passes;
    }
    const double cpu_us = spent / passes * 1e6;
    double max_diff = 0, num = 0, den = 0;
    for (size_t i = 0; i < Y.size(); ++i) {
        const double d = to_double(Y_gpu[i]) - (double)Y[i];
        max_diff = std::max(max_diff, std::fabs(d));
        num += d * d;
        den += (double)Y[i] * (double)Y[i];
    }
    const double rel = den > 0 ? std::sqrt(num / den) : std::sqrt(num);
    const double gflops = 2.0 * nnz * K / (cpu_us * 1e3);
    std::printf("cpu baseline: %.1f us per product (%.2f GFLOP/s) on %u of %u host threads, %d passes; device is %.1fx faster\n",
                cpu_us, gflops, threads, present, passes, gpu_us > 0 ? cpu_us / gpu_us : 0.0);
    std::printf("device against the cpu row loop: max |diff| %.3e, relative Frobenius %.3e\n", max_diff, rel);
    char buf[256];
    std::snprintf(buf, sizeof buf,
                  ", \"cpu_us\": %.1f, \"cpu_gflops\": %.3f, \"cpu_threads\": %u, \"cpu_threads_present\": %u, "
                  "\"max_abs_diff_vs_cpu\": %.3e, \"rel_fro_vs_cpu\": %.3e",
                  cpu_us, gflops, threads, present, max_diff, rel);
    return buf;
}

// <cost>: a number, or "default" / 0 for the library's choice (resolved once the graph is known)
inline int parse_cost(const std::string &s) { return s == "default" ? 0 : std::atoi(s.c_str()); }

}  // namespace drv
#endif
