// gather_probe
// What the memory system of the GPU gives a gather-scale-accumulate kernel,
// measured apart from the SpMM kernels: random rows of a dense table fetched
// the way mp_spmm_kernel fetches rows of X (ROW / 16 lanes per row, 16 bytes
// per lane, 8 rows in flight per lane), the table resident in the L2 of an XCD
// or far beyond it, alone or beside the sparse stream (8 bytes per nonzero,
// one coalesced non-temporal 1 KiB load per wavefront and 8 rows), and the
// same rows served from an LDS table by 1024-thread workgroups.  Every line
// ends with the time the rate would need for 114.6 M nonzeros (the benchmark's
// 232,965-row power-law graph), to set beside the measured kernel times.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                            \
    do {                                                                 \
        hipError_t e_ = (x);                                             \
        if (e_ != hipSuccess) {                                          \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); \
            std::exit(1);                                                \
        }                                                                \
    } while (0)

typedef float f4_t __attribute__((ext_vector_type(4)));
constexpr int kDepth = 8;  // rows in flight per lane

// LANES_LOG2: lanes per row (2 -> 64-byte rows, 3 -> 128-byte rows).
// LDS_ROWS > 0: rows come from an LDS copy of the first LDS_ROWS rows.
template <int LANES_LOG2, bool STREAM, int THREADS, bool FROM_LDS>
__global__ __launch_bounds__(THREADS) void probe_kernel(const f4_t *__restrict__ tab, unsigned row_mask,
                                                         const f4_t *__restrict__ stream, size_t stream_vec, int iters,
                                                         f4_t *__restrict__ out, unsigned seed, int lds_rows)
{
    extern __shared__ f4_t s_tab[];
    if (FROM_LDS) {
        for (int i = threadIdx.x; i < (lds_rows << LANES_LOG2); i += THREADS) s_tab[i] = tab[i];
        __syncthreads();
    }
    const size_t tid = (size_t)blockIdx.x * THREADS + threadIdx.x;
    const unsigned group = (unsigned)(tid >> LANES_LOG2);
    const int s = threadIdx.x & ((1 << LANES_LOG2) - 1);
    const size_t wave = tid >> 6;
    const int lane = threadIdx.x & 63;
    unsigned state = (group * 2654435761u) ^ seed;
    f4_t acc = 0;
    for (int it = 0; it < iters; ++it) {
        f4_t sv = 0;
        if (STREAM) sv = __builtin_nontemporal_load(stream + ((wave * iters + it) * 64 + lane) % stream_vec);
        f4_t x[kDepth];
#pragma unroll
        for (int j = 0; j < kDepth; ++j) {
            state = state * 1664525u + 1013904223u;
            const unsigned row = (state >> 8) & row_mask;
            x[j] = FROM_LDS ? s_tab[(row << LANES_LOG2) + s] : tab[((size_t)row << LANES_LOG2) + s];
        }
#pragma unroll
        for (int j = 0; j < kDepth; ++j) acc += x[j];
        acc += sv;
    }
    if (acc[0] == 12345.678f) out[group] = acc;  // never true: keeps the loads alive
}

template <int LANES_LOG2, bool STREAM, int THREADS, bool FROM_LDS>
void run(const char *what, const f4_t *tab, size_t table_bytes, const f4_t *stream, size_t stream_bytes, f4_t *out,
         int blocks, int iters)
{
    const unsigned row_bytes = 16u << LANES_LOG2;
    const unsigned rows = (unsigned)(table_bytes / row_bytes);  // a power of two
    const size_t lds = FROM_LDS ? table_bytes : 0;
    auto kern = probe_kernel<LANES_LOG2, STREAM, THREADS, FROM_LDS>;
    if (lds) CK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipEvent_t a, b;
    CK(hipEventCreate(&a));
    CK(hipEventCreate(&b));
    const int reps = 5;
    for (int r = -2; r < reps; ++r) {
        if (r == 0) CK(hipEventRecord(a));
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(THREADS), lds, 0, tab, rows - 1, stream, stream_bytes / 16, iters, out,
                           99u + r, (int)rows);
    }
    CK(hipEventRecord(b));
    CK(hipDeviceSynchronize());
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, a, b));
    ms /= reps;
    const double gathers = (double)blocks * THREADS / (1 << LANES_LOG2) * iters * kDepth;
    std::printf("%-58s %7.3f ms  %6.1f G rows/s  %5.2f TB/s of rows  114.6 M rows in %.3f ms\n", what, ms, gathers / ms / 1e6,
                gathers * row_bytes / ms / 1e9, 114.6e6 / (gathers / ms));
    CK(hipEventDestroy(a));
    CK(hipEventDestroy(b));
}

int main()
{
    f4_t *tab, *stream, *out;
    const size_t stream_bytes = 2ull << 30;
    CK(hipMalloc(&tab, 64ull << 20));
    CK(hipMemset(tab, 0, 64ull << 20));
    CK(hipMalloc(&stream, stream_bytes));
    CK(hipMemset(stream, 0, stream_bytes));
    CK(hipMalloc(&out, 64ull << 20));
    int cus = 256;
    CK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
    const int blocks = cus * 32;  // 256-thread workgroups, 8 resident per CU, 4 rounds
    run<2, false, 256, false>("64-byte rows, 2 MiB table (L2 of an XCD)", tab, 2ull << 20, stream, stream_bytes, out, blocks, 64);
    run<3, false, 256, false>("128-byte rows, 2 MiB table (L2 of an XCD)", tab, 2ull << 20, stream, stream_bytes, out, blocks, 64);
    run<2, false, 256, false>("64-byte rows, 64 MiB table (beyond L2)", tab, 64ull << 20, stream, stream_bytes, out, blocks, 64);
    run<3, false, 256, false>("128-byte rows, 64 MiB table (beyond L2)", tab, 64ull << 20, stream, stream_bytes, out, blocks, 64);
    run<2, true, 256, false>("64-byte rows, 2 MiB table + 8 B/row stream from HBM", tab, 2ull << 20, stream, stream_bytes, out, blocks,
                             64);
    run<2, true, 1024, true>("64-byte rows, 128 KiB LDS table + stream, 16 waves per CU", tab, 128ull << 10, stream, stream_bytes,
                             out, cus, 2048);
    run<2, false, 1024, true>("64-byte rows, 128 KiB LDS table, no stream", tab, 128ull << 10, stream, stream_bytes, out, cus, 2048);
    return 0;
}
