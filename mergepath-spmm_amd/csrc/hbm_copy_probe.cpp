// hbm_copy_probe [MiB] [repeats]
// A plain device-to-device copy kernel of known size.  Run under
// `rocprofv3 --pmc FETCH_SIZE` (then WRITE_SIZE) to learn what those counters
// read for a known number of HBM bytes; the SpMM kernels' counter readings are
// scaled by the same factor.  Two kernels: ordinary loads, and the
// non-temporal loads that the SpMM kernels use for the sparse stream.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));               \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

typedef float f4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void copy_plain_kernel(const f4_t *__restrict__ src, f4_t *__restrict__ dst, size_t n)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void copy_nontemporal_kernel(const f4_t *__restrict__ src, f4_t *__restrict__ dst,
                                                                size_t n)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = __builtin_nontemporal_load(src + i);
}

int main(int argc, char **argv)
{
    size_t mib = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 1024;
    int repeats = argc > 2 ? std::atoi(argv[2]) : 5;
    size_t bytes = mib << 20, n = bytes / sizeof(f4_t);
    f4_t *src = nullptr, *dst = nullptr;
    CK(hipMalloc(reinterpret_cast<void **>(&src), bytes));
    CK(hipMalloc(reinterpret_cast<void **>(&dst), bytes));
    CK(hipMemset(src, 1, bytes));
    CK(hipMemset(dst, 0, bytes));
    hipEvent_t a, b;
    CK(hipEventCreate(&a));
    CK(hipEventCreate(&b));
    for (int variant = 0; variant < 2; ++variant) {
        for (int r = -1; r < repeats; ++r) {
            if (r == 0) CK(hipEventRecord(a));
            if (variant == 0)
                hipLaunchKernelGGL(copy_plain_kernel, dim3(256 * 16), dim3(256), 0, 0, src, dst, n);
            else
                hipLaunchKernelGGL(copy_nontemporal_kernel, dim3(256 * 16), dim3(256), 0, 0, src, dst, n);
        }
        CK(hipEventRecord(b));
        CK(hipDeviceSynchronize());
        float ms = 0;
        CK(hipEventElapsedTime(&ms, a, b));
        ms /= repeats;
        std::printf("%s: %zu MiB read + %zu MiB written per launch, %.3f ms, %.1f GB/s (read+write)\n",
                    variant == 0 ? "copy_plain_kernel" : "copy_nontemporal_kernel", mib, mib, ms, 2.0 * bytes / ms / 1e6);
    }
    return 0;
}
