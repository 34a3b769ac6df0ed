// hot_launch_probe
// Synthetic model of the hot launch of a plan (rows of X in an LDS table, 16
// lane-groups of 4 lanes per wavefront, 1024-thread workgroups, one per CU),
// built up one feature at a time so that the cost of each can be read off:
//   gather      row slots from a generator in registers, nothing else
//   + stream    slots and values come from a sliced stream (2 KiB per
//               wavefront and round, non-temporal loads), staged through LDS
//   + row ends  one entry in 36 carries a row end; the finished row is
//               written to LDS only (the divergence, without the stores)
//   + stores    the finished row is written to global memory, with plain or
//               non-temporal stores (on this GPU a wait for a load also
//               waits for every older store)
// Same number of nonzeros as the hot columns of the benchmark's power-law
// graph hold (41.9 M per launch).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x)                                                            \
    do {                                                                 \
        hipError_t e_ = (x);                                             \
        if (e_ != hipSuccess) {                                          \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); \
            std::exit(1);                                                \
        }                                                                \
    } while (0)

typedef float f4_t __attribute__((ext_vector_type(4)));
typedef int i4_t __attribute__((ext_vector_type(4)));
constexpr int kWaves = 16;        // wavefronts per workgroup
constexpr int kRowsPerGroup = 64; // output rows reserved per lane-group (about 18 are used)

enum Mode { kGather = 0, kStream = 1, kRowEndsLds = 2, kRowEndsPlain = 3, kRowEndsNt = 4 };

__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int MODE>
__global__ __launch_bounds__(64 * kWaves) void probe_kernel(const f4_t *__restrict__ X, const int *__restrict__ cols,
                                                             const float *__restrict__ vals, int rounds,
                                                             f4_t *__restrict__ Y, int lds_rows, unsigned seed)
{
    extern __shared__ f4_t s_tab[];
    __shared__ int s_col[kWaves][256];
    __shared__ float s_val[kWaves][256];
    __shared__ f4_t s_out[kWaves][64];
    for (int i = threadIdx.x; i < lds_rows * 4; i += 64 * kWaves) s_tab[i] = X[i];
    __syncthreads();
    const int wib = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 2, s = lane & 3;
    const size_t wave = (size_t)blockIdx.x * kWaves + wib;
    const unsigned mask = lds_rows - 1;
    f4_t acc = 0;
    unsigned state = ((unsigned)(wave * 16 + g) * 2654435761u) ^ seed;
    size_t row_out = (wave * 16 + g) * kRowsPerGroup;
    const size_t row_stop = row_out + kRowsPerGroup - 1;  // never written past: the data has too few row ends for that
    const size_t base = wave * (size_t)rounds * 256;
    i4_t pc = __builtin_nontemporal_load(reinterpret_cast<const i4_t *>(cols + base + 4 * lane));
    f4_t pv = __builtin_nontemporal_load(reinterpret_cast<const f4_t *>(vals + base + 4 * lane));
    for (int r = 0; r < rounds; ++r) {
        if (MODE >= kStream) {
            *reinterpret_cast<i4_t *>(&s_col[wib][4 * lane]) = pc;
            *reinterpret_cast<f4_t *>(&s_val[wib][4 * lane]) = pv;
            wave_lds_sync();
        }
        if (r + 1 < rounds) {
            pc = __builtin_nontemporal_load(reinterpret_cast<const i4_t *>(cols + base + (size_t)(r + 1) * 256 + 4 * lane));
            pv = __builtin_nontemporal_load(reinterpret_cast<const f4_t *>(vals + base + (size_t)(r + 1) * 256 + 4 * lane));
        }
#pragma unroll
        for (int b = 0; b < 16; b += 4) {
            int ent[4];
            float av[4];
            f4_t x[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (MODE == kGather) {
                    state = state * 1664525u + 1013904223u;
                    ent[j] = (int)((state >> 8) & 0xffff);
                    av[j] = 1.0f;
                } else {
                    ent[j] = s_col[wib][g * 16 + b + j];
                    av[j] = s_val[wib][g * 16 + b + j];
                }
                x[j] = s_tab[((ent[j] & mask) << 2) + s];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (MODE >= kRowEndsLds) {
                    for (unsigned e = (unsigned)ent[j] >> 16; e != 0 && row_out < row_stop; --e) {
                        if (MODE == kRowEndsLds) s_out[wib][lane] = acc;
                        else if (MODE == kRowEndsNt) __builtin_nontemporal_store(acc, Y + row_out * 4 + s);
                        else Y[row_out * 4 + s] = acc;
                        ++row_out;
                        acc = 0;
                    }
                }
                acc += av[j] * x[j];
            }
        }
        if (MODE >= kStream) wave_lds_sync();
    }
    if (MODE == kRowEndsLds) acc += s_out[wib][lane];
    Y[row_out * 4 + s] = acc;
}

template <int MODE>
void run(const char *what, const f4_t *X, const int *cols, const float *vals, f4_t *Y, int blocks, int rounds, int lds_rows)
{
    const size_t lds = (size_t)lds_rows * 64;
    auto kern = probe_kernel<MODE>;
    CK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipEvent_t a, b;
    CK(hipEventCreate(&a));
    CK(hipEventCreate(&b));
    const int reps = 5;
    for (int r = -2; r < reps; ++r) {
        if (r == 0) CK(hipEventRecord(a));
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(64 * kWaves), lds, 0, X, cols, vals, rounds, Y, lds_rows, 99u + r);
    }
    CK(hipEventRecord(b));
    CK(hipDeviceSynchronize());
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, a, b));
    ms /= reps;
    const double nnz = (double)blocks * kWaves * rounds * 256;
    std::printf("%-44s %6.1f us for %.1f M nonzeros  %6.1f G/s\n", what, ms * 1e3, nnz / 1e6, nnz / ms / 1e6);
    CK(hipEventDestroy(a));
    CK(hipEventDestroy(b));
}

int main()
{
    int cus = 256;
    CK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
    const int blocks = cus, rounds = 40, lds_rows = 1024;
    const size_t n = (size_t)blocks * kWaves * rounds * 256;
    std::vector<int> h_cols(n);
    std::vector<float> h_vals(n, 0.5f);
    unsigned st = 12345;
    for (size_t i = 0; i < n; ++i) {  // one row end in 36 entries: the average row of the hot segments
        st = st * 1664525u + 1013904223u;
        const unsigned r = st >> 8;
        h_cols[i] = (int)((r >> 6) & 1023) | (((r % 36u) == 0) << 16);
    }
    const size_t y_bytes = (size_t)blocks * kWaves * 16 * kRowsPerGroup * 64;
    f4_t *X, *Y;
    int *cols;
    float *vals;
    CK(hipMalloc(&X, 1 << 20));
    CK(hipMemset(X, 0, 1 << 20));
    CK(hipMalloc(&Y, y_bytes));
    CK(hipMalloc(&cols, n * sizeof(int)));
    CK(hipMalloc(&vals, n * sizeof(float)));
    CK(hipMemcpy(cols, h_cols.data(), n * sizeof(int), hipMemcpyHostToDevice));
    CK(hipMemcpy(vals, h_vals.data(), n * sizeof(float), hipMemcpyHostToDevice));
    run<kGather>("gather from the LDS table", X, cols, vals, Y, blocks, rounds, lds_rows);
    run<kStream>("+ sliced stream staged through LDS", X, cols, vals, Y, blocks, rounds, lds_rows);
    run<kRowEndsLds>("+ row ends, finished rows to LDS", X, cols, vals, Y, blocks, rounds, lds_rows);
    run<kRowEndsPlain>("+ finished rows to memory, plain stores", X, cols, vals, Y, blocks, rounds, lds_rows);
    run<kRowEndsNt>("+ finished rows to memory, non-temporal", X, cols, vals, Y, blocks, rounds, lds_rows);
    return 0;
}
