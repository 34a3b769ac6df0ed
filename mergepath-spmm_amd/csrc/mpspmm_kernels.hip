// Device half of the MergePath-SpMM C ABI: hand-written HIP kernels for
// gfx950 (CDNA4, 64-lane wavefronts) and their launchers.
//
// Work decomposition.  A wavefront is cut into lane-groups of L = 4..64 lanes
// (L * VEC >= min(K, 64 * VEC) columns, VEC = one 16-byte load per lane where
// K allows).  In the merge-path kernel every lane-group walks one partition
// of the reference schedule (src/MergePathSpMM.cu:300-385): `cost` merge
// items = row ends + nonzeros.  The group streams its col_idx / val run
// through LDS in 16-nonzero windows (one 64-byte load per array per window,
// the next window prefetched into registers while the current one is
// consumed), gathers the 16 dense rows with 16-byte loads, and accumulates in
// fp32 registers.  Rows that end inside a partition after its first row end
// are stored directly.  A group's first finished row and its unfinished last
// row are partial: they are first combined across the groups of the
// wavefront through LDS, and what still crosses the wavefront boundary is
// written to a carry-out record that a second kernel folds in.  No atomics.
//
// Plans (mpspmm_plan.hip) run the same kernel over a column-slab tiled,
// sliced copy of the matrix.
#include "mpspmm_device.hpp"

#include <mutex>

namespace {

// ---------------------------------------------------------------------------
// Merge-path partitioner: MergePathSearch (src/MergePathSpMM.cu:280-297) on
// the diagonals of generate_mp_sched (:327-334), one thread per boundary.
// NZ_INDICES[i] == i (:311-313) is not materialised: NZ_INDICES[d - pivot - 1]
// is d - pivot - 1.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void mp_partition_kernel(const int *__restrict__ row_ptr, int num_rows,
                                                            int nnz, int P, int ipt,
                                                            int *__restrict__ coord_x,
                                                            int *__restrict__ coord_y)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i > P) return;
    const int total = num_rows + nnz;
    long long d64 = (long long)ipt * i;
    int diagonal = d64 < (long long)total ? (int)d64 : total;
    int x_min = max(diagonal - nnz, 0);
    int x_max = min(diagonal, num_rows);
    while (x_min < x_max) {
        int pivot = (x_min + x_max) >> 1;
        if (row_ptr[pivot] <= diagonal - pivot - 1)
            x_min = pivot + 1;
        else
            x_max = pivot;
    }
    coord_x[i] = min(x_min, num_rows);
    coord_y[i] = diagonal - x_min;
}

// The six per-partition arrays that generate_mp_sched hands to the reference
// kernels (src/MergePathSpMM.cu:336-376), derived from the boundary
// coordinates.  Partition i covers rows first..last; it has a head piece when
// it starts inside row `first` (its first nonzero, y_begin, is not the row's
// first one) and a tail piece when it stops inside row `last`.  The reference
// stores a piece as (nonzero index, count) and writes index 0 for "no piece",
// so a piece that would start at nonzero 0 is reported as absent; partition 0
// never has a head.  A partition that lies inside a single row is all head.
__global__ __launch_bounds__(256) void mp_schedule_legacy_kernel(
    const int *__restrict__ row_ptr, int P, const int *__restrict__ coord_x,
    const int *__restrict__ coord_y, int *__restrict__ head_at_out, int *__restrict__ head_count_out,
    int *__restrict__ tail_at_out, int *__restrict__ tail_count_out, int *__restrict__ first_row_out,
    int *__restrict__ last_row_out)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= P) return;
    const int first = max(coord_x[i] - 1, 0), last = coord_x[i + 1] - 1;
    const int y_begin = coord_y[i], y_end = coord_y[i + 1];
    const int last_begin = row_ptr[last];
    const bool head = i != 0 && y_begin != row_ptr[first] && y_begin != 0;
    bool tail = y_end != last_begin && y_end != 0;
    const bool one_row = head && tail && first == last;
    int head_count = 0;
    if (head) head_count = (one_row ? y_end : row_ptr[first + 1]) - y_begin;
    if (one_row) tail = false;
    head_at_out[i] = head ? y_begin : 0;
    head_count_out[i] = head_count;
    tail_at_out[i] = tail ? last_begin : 0;
    tail_count_out[i] = tail ? y_end - last_begin : 0;
    first_row_out[i] = first;
    last_row_out[i] = last;
}

// ---------------------------------------------------------------------------
// One lane-group accumulates the nonzero range [y_begin, y_end) of one row.
// Wave-uniform control flow: every group of the wave runs the same number of
// rounds, idle ones with an empty range.
// ---------------------------------------------------------------------------
template <typename T, int VEC, bool POW2, int BATCH>
__device__ __forceinline__ void accumulate_range(const int *__restrict__ col_idx,
                                                 const T *__restrict__ val, const Gather<T, VEC, POW2> &gx,
                                                 int nnz, int y_begin, int y_end, int s, int *s_col,
                                                 float *s_val, float (&acc)[VEC])
{
    using XO = XOps<T, VEC>;
    using Raw = typename XO::Raw;
    int wbase = y_begin;
    Win pw;
    pw.c = make_int4(0, 0, 0, 0);
    pw.v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (s < 4 && wbase < y_end) pw = load_win<T>(col_idx, val, nnz, wbase + 4 * s);
    while (__any(wbase < y_end)) {
        const int nvalid = min(kWindow, y_end - wbase);
        if (s < 4 && nvalid > 0) {
            *reinterpret_cast<int4 *>(s_col + 4 * s) = pw.c;
            *reinterpret_cast<float4 *>(s_val + 4 * s) = pw.v;
        }
        wave_lds_sync();
#pragma unroll
        for (int b = 0; b < kWindow; b += BATCH) {
            int cols[BATCH];
            float vals[BATCH];
            Raw xr[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                cols[j] = s_col[b + j];
                vals[j] = s_val[b + j];
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j)
                if (b + j < nvalid) xr[j] = gx.load(cols[j]);
            if (b == 0) {
                const int nb = wbase + kWindow;
                if (s < 4 && nb < y_end) pw = load_win<T>(col_idx, val, nnz, nb + 4 * s);
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j)
                if (b + j < nvalid) XO::fma(acc, vals[j], xr[j]);
        }
        wbase += kWindow;
        wave_lds_sync();
    }
}

// Row-wise comparison kernel (src/row_wise.cu:194-240): wavefront w owns the
// rows [int(step * w), int(step * (w + 1))); its lane-groups take those rows
// round-robin, one whole row per group, plain stores.
template <typename T, int VEC, bool POW2, int BATCH>
__global__ __launch_bounds__(kBlock) void rowwise_spmm_kernel(
    const int *__restrict__ row_ptr, const int *__restrict__ col_idx, const T *__restrict__ val,
    const T *__restrict__ X, T *__restrict__ Y, int n_rows, int nnz, int K, int lanes_log2,
    int num_waves, int row_shift, float step)
{
    __shared__ float s_buf[kWavesPerBlock][2 * 16 * kWindow];
    const int wib = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int w = blockIdx.x * kWavesPerBlock + wib;
    if (w >= num_waves) return;
    const int L = 1 << lanes_log2;
    const int G = 64 >> lanes_log2;
    const int g = lane >> lanes_log2;
    const int s = lane & (L - 1);
    const int KT = L * VEC;
    const int kcol = blockIdx.y * KT + s * VEC;
    const bool col_ok = kcol < K;
    const Gather<T, VEC, POW2> gx{reinterpret_cast<const char *>(X), (size_t)K * sizeof(T),
                                  col_ok ? (unsigned)(kcol * sizeof(T)) : 0u, row_shift};
    int *s_col = reinterpret_cast<int *>(&s_buf[wib][0]) + g * kWindow;
    float *s_val = &s_buf[wib][16 * kWindow] + g * kWindow;

    int row_start = min((int)(step * (float)w), n_rows);
    int row_stop = (w == num_waves - 1) ? n_rows : min((int)(step * (float)(w + 1)), n_rows);

    for (int r0 = row_start; r0 < row_stop; r0 += G) {
        const int row = r0 + g;
        const bool row_ok = row < row_stop;
        int y_begin = 0, y_end = 0;
        if (row_ok) {
            y_begin = row_ptr[row];
            y_end = row_ptr[row + 1];
        }
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        accumulate_range<T, VEC, POW2, BATCH>(col_idx, val, gx, nnz, y_begin, y_end, s, s_col, s_val, acc);
        if (row_ok && col_ok) store_acc<VEC>(Y + (size_t)row * K + kcol, acc);
    }
}

// Nonzero-splitting comparison kernel (src/nz_splitting.cu:318-445): one
// group of at most part_size nonzeros per lane-group, ending in atomic adds.
template <typename T, int VEC, bool POW2, int BATCH>
__global__ __launch_bounds__(kBlock) void nzsplit_spmm_kernel(
    const int *__restrict__ col_idx, const T *__restrict__ val, const T *__restrict__ X,
    float *__restrict__ Y, int nnz, int K, int lanes_log2, int row_shift,
    const int *__restrict__ part_ptr, const int *__restrict__ part2node, int num_parts, int num_waves)
{
    __shared__ float s_buf[kWavesPerBlock][2 * 16 * kWindow];
    const int wib = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int w = blockIdx.x * kWavesPerBlock + wib;
    if (w >= num_waves) return;
    const int L = 1 << lanes_log2;
    const int G = 64 >> lanes_log2;
    const int g = lane >> lanes_log2;
    const int s = lane & (L - 1);
    const int KT = L * VEC;
    const int kcol = blockIdx.y * KT + s * VEC;
    const bool col_ok = kcol < K;
    const Gather<T, VEC, POW2> gx{reinterpret_cast<const char *>(X), (size_t)K * sizeof(T),
                                  col_ok ? (unsigned)(kcol * sizeof(T)) : 0u, row_shift};
    int *s_col = reinterpret_cast<int *>(&s_buf[wib][0]) + g * kWindow;
    float *s_val = &s_buf[wib][16 * kWindow] + g * kWindow;

    const int part = w * G + g;
    const bool part_ok = part < num_parts;
    int y_begin = 0, y_end = 0, row = 0;
    if (part_ok) {
        y_begin = part_ptr[part];
        y_end = part_ptr[part + 1];
        row = part2node[part];
    }
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    accumulate_range<T, VEC, POW2, BATCH>(col_idx, val, gx, nnz, y_begin, y_end, s, s_col, s_val, acc);
    if (part_ok && col_ok) {
        float *y = Y + (size_t)row * K + kcol;
#pragma unroll
        for (int i = 0; i < VEC; ++i) unsafeAtomicAdd(y + i, acc[i]);
    }
}

__global__ __launch_bounds__(256) void fill_zero_kernel(float4 *__restrict__ p4, size_t n4,
                                                         float *__restrict__ tail, int ntail)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t j = i; j < n4; j += stride) p4[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < (size_t)ntail) tail[i] = 0.f;
}

// ---------------------------------------------------------------------------
// nz-splitting plan (src/nz_splitting.cu:256-316) on the device.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void nzsplit_count_kernel(const int *__restrict__ row_ptr, int n_rows,
                                                             int part_size, int *__restrict__ counts)
{
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r > n_rows) return;
    int c = 0;
    if (r < n_rows) {
        int degree = row_ptr[r + 1] - row_ptr[r];
        c = degree / part_size + (degree % part_size != 0);
    }
    counts[r] = c;
}

// One thread per group: find its row by binary search in the offsets.
__global__ __launch_bounds__(256) void nzsplit_fill_kernel(const int *__restrict__ row_ptr,
                                                            const int *__restrict__ offsets, int n_rows,
                                                            int part_size, int max_parts,
                                                            int *__restrict__ part_ptr,
                                                            int *__restrict__ part2node)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    const int num_parts = offsets[n_rows];
    if (t == 0 && num_parts <= max_parts) part_ptr[num_parts] = row_ptr[n_rows];
    if (t >= num_parts || t >= max_parts) return;
    int lo = 0, hi = n_rows;  // largest r with offsets[r] <= t
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (offsets[mid] <= t) lo = mid; else hi = mid - 1;
    }
    const int pid = t - offsets[lo];
    part_ptr[t] = row_ptr[lo] + pid * part_size;
    part2node[t] = lo;
}

// ---------------------------------------------------------------------------
// CSR validation
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void csr_validate_kernel(const int *__restrict__ row_ptr,
                                                            const int *__restrict__ col_idx, int n_rows,
                                                            int n_cols, int nnz, int *__restrict__ bad)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    int err = 0;
    for (size_t r = i; r <= (size_t)n_rows; r += stride) {
        int v = row_ptr[r];
        if (r == 0 && v != 0) err = 1;
        if (r == (size_t)n_rows && v != nnz) err = 1;
        if (r < (size_t)n_rows && row_ptr[r + 1] < v) err = 1;
        if (v < 0 || v > nnz) err = 1;
    }
    for (size_t e = i; e < (size_t)nnz; e += stride) {
        int c = col_idx[e];
        if (c < 0 || c >= n_cols) err = 1;
    }
    if (err) atomicOr(bad, 1);
}

// ---------------------------------------------------------------------------
// Edge weights from degrees: the reference's implicit weight, written out.
// degrees[i] = row_ptr[i + 1] - row_ptr[i] (src/MergePathSpMM.cu:183-185);
// weight of nonzero (r, c) = float(deg r) * float(deg c), one rounded product
// (__fmaf_rn(a, b, 0), :450,459); the fp16 program multiplies the two degrees
// converted to half, in half (src/MergePathSpMM_fp16.cu:451,460), which
// overflows to infinity beyond 65504.  MPS_WEIGHT_GCN is the normalisation
// GCN layers use, 1 / sqrt(deg r * deg c), 0 where a degree is 0.
// One thread per nonzero; its row is found by bisection of row_ptr.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void degree_values_kernel(const int *__restrict__ row_ptr,
                                                             const int *__restrict__ col_idx, int n_rows, int nnz,
                                                             int mode, T *__restrict__ val)
{
    const long long e64 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e64 >= nnz) return;
    const int e = (int)e64;
    int lo = 0, hi = n_rows - 1;  // largest r with row_ptr[r] <= e
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (row_ptr[mid] <= e) lo = mid; else hi = mid - 1;
    }
    const int c = col_idx[e];
    const int dr = row_ptr[lo + 1] - row_ptr[lo];
    const int dc = row_ptr[c + 1] - row_ptr[c];
    if (mode == MPS_WEIGHT_GCN) {
        const float p = (float)dr * (float)dc;
        val[e] = (T)(p > 0.f ? 1.0f / sqrtf(p) : 0.f);
    } else {
        val[e] = (T)dr * (T)dc;  // T = float: rounded fp32 product; T = half: both factors and the product in half
    }
}

template <typename T>
int degree_values_entry(const int *row_ptr, const int *col_idx, int n_rows, int nnz, int mode, T *val, void *stream)
{
    if (!row_ptr || n_rows < 0 || nnz < 0 || (nnz > 0 && (!col_idx || !val))) return MPS_ERR_INVALID_ARG;
    if (mode != MPS_WEIGHT_DEGREE_PRODUCT && mode != MPS_WEIGHT_GCN) return MPS_ERR_INVALID_ARG;
    if (nnz == 0) return MPS_OK;
    hipLaunchKernelGGL((degree_values_kernel<T>), dim3((unsigned)(((long long)nnz + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), row_ptr, col_idx, n_rows, nnz, mode, val);
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

template <typename T>
int check_spmm_args(const int *row_ptr, const int *col_idx, const T *val, const T *X, const void *Y, int n_rows,
                    long long n_vrows, int nnz, int K, int P, const int *cx, const int *cy)
{
    if (n_rows < 0 || nnz < 0 || K < 1 || P < 1) return MPS_ERR_INVALID_ARG;
    if (!row_ptr || !cx || !cy || (nnz > 0 && (!col_idx || !val))) return MPS_ERR_INVALID_ARG;
    if (n_rows > 0 && (!X || !Y)) return MPS_ERR_INVALID_ARG;
    if (n_vrows + 1 + nnz > INT_MAX) return MPS_ERR_UNSUPPORTED;
    if ((long long)P > INT_MAX / 2) return MPS_ERR_UNSUPPORTED;
    if (!aligned_to(col_idx, 4) || !aligned_to(val, sizeof(T)) || !aligned_to(X, 16) || !aligned_to(Y, 16))
        return MPS_ERR_ALIGNMENT;
    return MPS_OK;
}

template <typename T>
int spmm_entry(const int *row_ptr, const int *col_idx, const T *val, const T *X, T *Y, int n_rows, int nnz, int K,
               int P, const int *cx, const int *cy, int tpw, void *ws, size_t ws_bytes, unsigned phases,
               void *stream)
{
    int rc = check_spmm_args<T>(row_ptr, col_idx, val, X, Y, n_rows, n_rows, nnz, K, P, cx, cy);
    if (rc != MPS_OK) return rc;
    SpmmShape sh;
    rc = make_spmm_shape(n_rows, K, P, tpw, (int)sizeof(T), sh);
    if (rc != MPS_OK) return rc;
    if (!ws || ws_bytes < carry_bytes_for(sh.num_waves, K)) return MPS_ERR_WORKSPACE;
    if (!aligned_to(ws, 16)) return MPS_ERR_ALIGNMENT;
    return launch_spmm_any<T, T>(row_ptr, col_idx, val, X, Y, nnz, K, P, cx, cy, PlanLaunch{}, sh, ws, phases,
                                 static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------
// Carry-out records in device memory that the library never allocates: a
// file-scope array, one copy per GPU, for callers that must not call hipMalloc.
// `scratch` is a host-side stand-in for the array; its device address is looked
// up once per device (hipGetSymbolAddress) and only that address is handed to
// kernels.
// ---------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = (size_t)MPS_STATIC_SCRATCH_MIB << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxDevices];  // per device, nullptr until first use there

int static_scratch(void **ptr_out)
{
    int dev = 0;
    MPS_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return MPS_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        MPS_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return MPS_ERR_HIP + (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
    }
    *ptr_out = g_scratch_ptr[dev];
    return MPS_OK;
}

}  // namespace

// ===========================================================================
// C ABI
// ===========================================================================
extern "C" {

int mps_csr_validate(const int *d_row_ptr, const int *d_col_idx, int n_rows, int n_cols, int nnz,
                     void *stream)
{
    if (!d_row_ptr || n_rows < 0 || n_cols < 0 || nnz < 0 || (nnz > 0 && !d_col_idx))
        return MPS_ERR_INVALID_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int *d_bad = nullptr;
    MPS_HIP_TRY(hipMalloc(&d_bad, sizeof(int)));
    int zero = 0, bad = 0;
    hipError_t e = hipMemcpyAsync(d_bad, &zero, sizeof(int), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) {
        size_t work = (size_t)nnz > (size_t)n_rows + 1 ? (size_t)nnz : (size_t)n_rows + 1;
        unsigned blocks = (unsigned)((work + 255) / 256);
        if (blocks > 16384) blocks = 16384;
        if (blocks < 1) blocks = 1;
        hipLaunchKernelGGL(csr_validate_kernel, dim3(blocks), dim3(256), 0, st, d_row_ptr, d_col_idx,
                           n_rows, n_cols, nnz, d_bad);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(&bad, d_bad, sizeof(int), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    hipError_t e2 = hipFree(d_bad);
    if (e != hipSuccess) return MPS_ERR_HIP + (int)e;
    if (e2 != hipSuccess) return MPS_ERR_HIP + (int)e2;
    return bad ? MPS_ERR_INVALID_CSR : MPS_OK;
}

int mps_degree_values_f32(const int *d_row_ptr, const int *d_col_idx, int n_rows, int nnz, int mode, float *d_val,
                          void *stream)
{
    return degree_values_entry<float>(d_row_ptr, d_col_idx, n_rows, nnz, mode, d_val, stream);
}

int mps_degree_values_f16(const int *d_row_ptr, const int *d_col_idx, int n_rows, int nnz, int mode, void *d_val,
                          void *stream)
{
    return degree_values_entry<half_t>(d_row_ptr, d_col_idx, n_rows, nnz, mode, static_cast<half_t *>(d_val), stream);
}

int mps_partition(const int *d_row_ptr, int n_rows, int nnz, int P, int *d_coord_x, int *d_coord_y,
                  void *stream)
{
    if (!d_row_ptr || !d_coord_x || !d_coord_y || n_rows < 0 || nnz < 0 || P < 1) return MPS_ERR_INVALID_ARG;
    long long total = (long long)n_rows + 1 + nnz;
    if (total > INT_MAX || P == INT_MAX) return MPS_ERR_UNSUPPORTED;
    int ipt = (int)((total + P - 1) / P);
    unsigned blocks = (unsigned)(((long long)P + 1 + 255) / 256);
    hipLaunchKernelGGL(mp_partition_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       d_row_ptr, n_rows + 1, nnz, P, ipt, d_coord_x, d_coord_y);
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

int mps_schedule_legacy(const int *d_row_ptr, int n_rows, int nnz, int P, const int *d_coord_x,
                        const int *d_coord_y, int *d_feature_start, int *d_feature_start_num,
                        int *d_feature_end, int *d_feature_end_num, int *d_start_row, int *d_end_row,
                        void *stream)
{
    if (!d_row_ptr || !d_coord_x || !d_coord_y || !d_feature_start || !d_feature_start_num ||
        !d_feature_end || !d_feature_end_num || !d_start_row || !d_end_row)
        return MPS_ERR_INVALID_ARG;
    if (n_rows < 0 || nnz < 0 || P < 1) return MPS_ERR_INVALID_ARG;
    unsigned blocks = (unsigned)(((long long)P + 255) / 256);
    hipLaunchKernelGGL(mp_schedule_legacy_kernel, dim3(blocks), dim3(256), 0,
                       static_cast<hipStream_t>(stream), d_row_ptr, P, d_coord_x, d_coord_y,
                       d_feature_start, d_feature_start_num, d_feature_end, d_feature_end_num, d_start_row,
                       d_end_row);
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

int mps_spmm_workspace_bytes(int P, int K, int tpw, int elem_bytes, size_t *bytes_out)
{
    if (!bytes_out || (elem_bytes != 4 && elem_bytes != 2)) return MPS_ERR_INVALID_ARG;
    SpmmShape sh;
    int rc = make_spmm_shape(1, K, P, tpw, elem_bytes, sh);
    if (rc != MPS_OK) return rc;
    *bytes_out = carry_bytes_for(sh.num_waves, K);
    return MPS_OK;
}

int mps_spmm_f32_phases(const int *d_row_ptr, const int *d_col_idx, const float *d_val, const float *d_X,
                        float *d_Y, int n_rows, int nnz, int K, int P, const int *d_coord_x,
                        const int *d_coord_y, int tpw, void *d_workspace, size_t workspace_bytes,
                        unsigned phases, void *stream)
{
    return spmm_entry<float>(d_row_ptr, d_col_idx, d_val, d_X, d_Y, n_rows, nnz, K, P, d_coord_x, d_coord_y,
                             tpw, d_workspace, workspace_bytes, phases, stream);
}

int mps_spmm_f32(const int *d_row_ptr, const int *d_col_idx, const float *d_val, const float *d_X,
                 float *d_Y, int n_rows, int nnz, int K, int P, const int *d_coord_x, const int *d_coord_y,
                 int tpw, void *d_workspace, size_t workspace_bytes, void *stream)
{
    return spmm_entry<float>(d_row_ptr, d_col_idx, d_val, d_X, d_Y, n_rows, nnz, K, P, d_coord_x, d_coord_y,
                             tpw, d_workspace, workspace_bytes, MPS_PHASE_MAIN | MPS_PHASE_FIXUP, stream);
}

int mps_static_scratch_bytes(size_t *bytes_out)
{
    if (!bytes_out) return MPS_ERR_INVALID_ARG;
    *bytes_out = kStaticScratchBytes;
    return MPS_OK;
}

int mps_spmm_f32_static(const int *d_row_ptr, const int *d_col_idx, const float *d_val, const float *d_X,
                        float *d_Y, int n_rows, int nnz, int K, int P, const int *d_coord_x,
                        const int *d_coord_y, int tpw, void *stream)
{
    // sizes first: a request beyond the array must fail before anything touches the device
    SpmmShape sh;
    int rc = make_spmm_shape(n_rows > 0 ? n_rows : 1, K, P, tpw, 4, sh);
    if (rc != MPS_OK) return rc;
    if (carry_bytes_for(sh.num_waves, K) > kStaticScratchBytes) return MPS_ERR_WORKSPACE;
    void *ws = nullptr;
    if ((rc = static_scratch(&ws)) != MPS_OK) return rc;
    return spmm_entry<float>(d_row_ptr, d_col_idx, d_val, d_X, d_Y, n_rows, nnz, K, P, d_coord_x, d_coord_y,
                             tpw, ws, kStaticScratchBytes, MPS_PHASE_MAIN | MPS_PHASE_FIXUP, stream);
}

int mps_spmm_f16_phases(const int *d_row_ptr, const int *d_col_idx, const uint16_t *d_val,
                        const uint16_t *d_X, uint16_t *d_Y, int n_rows, int nnz, int K, int P,
                        const int *d_coord_x, const int *d_coord_y, int tpw, void *d_workspace,
                        size_t workspace_bytes, unsigned phases, void *stream)
{
    return spmm_entry<half_t>(d_row_ptr, d_col_idx, reinterpret_cast<const half_t *>(d_val),
                              reinterpret_cast<const half_t *>(d_X), reinterpret_cast<half_t *>(d_Y), n_rows,
                              nnz, K, P, d_coord_x, d_coord_y, tpw, d_workspace, workspace_bytes, phases,
                              stream);
}

int mps_spmm_f16(const int *d_row_ptr, const int *d_col_idx, const uint16_t *d_val, const uint16_t *d_X,
                 uint16_t *d_Y, int n_rows, int nnz, int K, int P, const int *d_coord_x,
                 const int *d_coord_y, int tpw, void *d_workspace, size_t workspace_bytes, void *stream)
{
    return mps_spmm_f16_phases(d_row_ptr, d_col_idx, d_val, d_X, d_Y, n_rows, nnz, K, P, d_coord_x,
                               d_coord_y, tpw, d_workspace, workspace_bytes,
                               MPS_PHASE_MAIN | MPS_PHASE_FIXUP, stream);
}

// ---- comparison kernels -----------------------------------------------------

int mps_rowwise_bounds(int n_rows, int num_waves, int *row_start, int *row_end)
{
    if (n_rows < 0 || num_waves < 1 || !row_start || !row_end) return MPS_ERR_INVALID_ARG;
    // float arithmetic of src/row_wise.cu:211-213
    float step = (float)n_rows / (float)num_waves;
    for (int w = 0; w < num_waves; ++w) {
        int a = (int)(step * (float)w);
        int b = (int)(step * (float)(w + 1));
        if (a > n_rows) a = n_rows;
        if (b > n_rows) b = n_rows;
        if (w == num_waves - 1) b = n_rows;
        row_start[w] = a;
        row_end[w] = b;
    }
    return MPS_OK;
}

int mps_rowwise_spmm_f32(const int *d_row_ptr, const int *d_col_idx, const float *d_val, const float *d_X,
                         float *d_Y, int n_rows, int nnz, int K, int num_waves, void *stream)
{
    if (n_rows < 0 || nnz < 0 || K < 1 || num_waves < 1 || !d_row_ptr) return MPS_ERR_INVALID_ARG;
    if (nnz > 0 && (!d_col_idx || !d_val)) return MPS_ERR_INVALID_ARG;
    if (n_rows > 0 && (!d_X || !d_Y)) return MPS_ERR_INVALID_ARG;
    if (!aligned_to(d_col_idx, 4) || !aligned_to(d_val, 4) || !aligned_to(d_X, 16) || !aligned_to(d_Y, 16))
        return MPS_ERR_ALIGNMENT;
    if (n_rows == 0) return MPS_OK;
    mps_lane_shape ls = mps_make_lane_shape(K, 4);
    const int row_shift = pow2_row_shift(n_rows, K, 4);
    float step = (float)n_rows / (float)num_waves;
    dim3 grid((num_waves + kWavesPerBlock - 1) / kWavesPerBlock, ls.col_tiles);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define MPS_LAUNCH_ROWWISE(VEC, POW2)                                                                     \
    hipLaunchKernelGGL((rowwise_spmm_kernel<float, VEC, POW2, 4>), grid, dim3(kBlock), 0, st, d_row_ptr,  \
                       d_col_idx, d_val, d_X, d_Y, n_rows, nnz, K, ls.lanes_log2, num_waves, row_shift, step)
    if (ls.vec == 4) { if (row_shift >= 0) MPS_LAUNCH_ROWWISE(4, true); else MPS_LAUNCH_ROWWISE(4, false); }
    else { if (row_shift >= 0) MPS_LAUNCH_ROWWISE(1, true); else MPS_LAUNCH_ROWWISE(1, false); }
#undef MPS_LAUNCH_ROWWISE
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

int mps_nzsplit_max_parts(int n_rows, int nnz, int part_size, int *max_parts_out)
{
    if (!max_parts_out || n_rows < 0 || nnz < 0 || part_size < 1) return MPS_ERR_INVALID_ARG;
    long long m = (long long)nnz / part_size + n_rows;
    if (m > INT_MAX - 1) return MPS_ERR_UNSUPPORTED;
    *max_parts_out = (int)m;
    return MPS_OK;
}

int mps_nzsplit_build(const int *d_row_ptr, int n_rows, int part_size, int *d_part_ptr, int *d_part2node,
                      int max_parts, int *d_scratch, int *num_parts_out, void *stream)
{
    if (!d_row_ptr || !d_part_ptr || !d_part2node || !d_scratch || !num_parts_out) return MPS_ERR_INVALID_ARG;
    if (n_rows < 0 || part_size < 1 || max_parts < 0) return MPS_ERR_INVALID_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int n = n_rows + 1;
    int *offsets = d_scratch;   // [n_rows + 1]
    int *sums = d_scratch + n;  // [2048]
    hipLaunchKernelGGL(nzsplit_count_kernel, dim3((n + 255) / 256), dim3(256), 0, st, d_row_ptr, n_rows, part_size,
                       offsets);
    MPS_HIP_TRY(hipGetLastError());
    int rc = scan_exclusive_inplace(offsets, n, sums, st);
    if (rc != MPS_OK) return rc;
    unsigned blocks = (unsigned)(((long long)max_parts + 255) / 256);
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(nzsplit_fill_kernel, dim3(blocks), dim3(256), 0, st, d_row_ptr, offsets, n_rows,
                       part_size, max_parts, d_part_ptr, d_part2node);
    MPS_HIP_TRY(hipGetLastError());
    int num_parts = 0;
    MPS_HIP_TRY(hipMemcpyAsync(&num_parts, offsets + n_rows, sizeof(int), hipMemcpyDeviceToHost, st));
    MPS_HIP_TRY(hipStreamSynchronize(st));
    *num_parts_out = num_parts;
    if (num_parts > max_parts) return MPS_ERR_WORKSPACE;
    return MPS_OK;
}

int mps_nzsplit_spmm_f32(const int *d_col_idx, const float *d_val, const float *d_X, float *d_Y, int n_rows,
                         int nnz, int K, const int *d_part_ptr, const int *d_part2node, int num_parts,
                         void *stream)
{
    if (n_rows < 0 || nnz < 0 || K < 1 || num_parts < 0) return MPS_ERR_INVALID_ARG;
    if (n_rows > 0 && (!d_X || !d_Y)) return MPS_ERR_INVALID_ARG;
    if (num_parts > 0 && (!d_part_ptr || !d_part2node || !d_col_idx || !d_val)) return MPS_ERR_INVALID_ARG;
    if (!aligned_to(d_col_idx, 4) || !aligned_to(d_val, 4) || !aligned_to(d_X, 16) || !aligned_to(d_Y, 16))
        return MPS_ERR_ALIGNMENT;
    if (n_rows == 0) return MPS_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    size_t total = (size_t)n_rows * K;
    size_t n4 = total / 4;
    int ntail = (int)(total - n4 * 4);
    unsigned zb = (unsigned)((n4 + 255) / 256);
    if (zb > 8192) zb = 8192;
    if (zb < 1) zb = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(zb), dim3(256), 0, st, reinterpret_cast<float4 *>(d_Y), n4,
                       d_Y + n4 * 4, ntail);
    MPS_HIP_TRY(hipGetLastError());
    if (num_parts == 0) return MPS_OK;
    mps_lane_shape ls = mps_make_lane_shape(K, 4);
    const int row_shift = pow2_row_shift(n_rows, K, 4);
    int num_waves = (num_parts + ls.groups - 1) / ls.groups;
    dim3 grid((num_waves + kWavesPerBlock - 1) / kWavesPerBlock, ls.col_tiles);
#define MPS_LAUNCH_NZSPLIT(VEC, POW2)                                                                    \
    hipLaunchKernelGGL((nzsplit_spmm_kernel<float, VEC, POW2, 4>), grid, dim3(kBlock), 0, st, d_col_idx, \
                       d_val, d_X, d_Y, nnz, K, ls.lanes_log2, row_shift, d_part_ptr, d_part2node,       \
                       num_parts, num_waves)
    if (ls.vec == 4) { if (row_shift >= 0) MPS_LAUNCH_NZSPLIT(4, true); else MPS_LAUNCH_NZSPLIT(4, false); }
    else { if (row_shift >= 0) MPS_LAUNCH_NZSPLIT(1, true); else MPS_LAUNCH_NZSPLIT(1, false); }
#undef MPS_LAUNCH_NZSPLIT
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

}  // extern "C"
