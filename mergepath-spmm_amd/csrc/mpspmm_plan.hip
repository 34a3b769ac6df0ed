// Plans: the per-matrix preprocessing of the merge-path SpMM, the counterpart
// of generate_mp_sched (src/MergePathSpMM.cu:192, :300-385), which the
// reference also runs once per matrix, outside its repeat loop.
//
// A plan holds
//   1. optionally, a column-slab tiled copy of the matrix: the nonzeros in
//      slab-major order, num_slabs * n_rows "virtual rows", so that the
//      running wavefronts gather from one ~3 MiB slab of X at a time (the L2
//      of an XCD is 4 MiB);
//   2. the merge-path partition of the (virtual) rows, from mps_partition;
//   3. the nonzeros "sliced" by that partition: the 16-nonzero windows that
//      the lane-groups of one wavefront consume in the same round are stored
//      side by side, so a wavefront stages a round with one contiguous load
//      per array (full 128-byte requests instead of one 64-byte piece per
//      group);
//   4. the workspace of the SpMM (per-slab partial rows, carry-out records).
#include "mpspmm_device.hpp"

struct mps_plan {
    int n_rows = 0, nnz = 0, K = 0, elem_bytes = 0, cost = 0;
    int num_slabs = 1, slab_cols = 0;
    int n_vrows = 0;
    int P = 0;
    SpmmShape shape{};
    long long total_rounds = 0;
    int *vrow_ptr = nullptr;
    int *coord_x = nullptr, *coord_y = nullptr;
    int *wave_off = nullptr;
    int *slice_cols = nullptr;
    void *slice_vals = nullptr;
    int *slice_src = nullptr;
    void *workspace = nullptr;
    size_t part_bytes = 0, workspace_bytes = 0;
    size_t device_bytes = 0;
};

namespace {

// Slab of X that stays resident in a 4 MiB L2 next to the streamed data
// (3 MiB measured best on the power-law benchmark graph; 2 and 2.5 MiB within 5 %).
constexpr size_t kDefaultSlabBytes = 3u << 20;

// ---------------------------------------------------------------------------
// Column-slab tiling plan.
// ---------------------------------------------------------------------------
// first[s * n_rows + r] = index of the first nonzero of row r whose column is
// >= s * slab_cols; counts[...] = number of nonzeros of row r in slab s.
__global__ __launch_bounds__(256) void tile_count_kernel(const int *__restrict__ row_ptr,
                                                          const int *__restrict__ col_idx, int n_rows,
                                                          int num_slabs, int slab_cols, int *__restrict__ first,
                                                          int *__restrict__ counts)
{
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long nv = (long long)num_slabs * n_rows;
    if (t == nv) counts[nv] = 0;
    if (t >= nv) return;
    const int s = (int)(t / n_rows);
    const int r = (int)(t - (long long)s * n_rows);
    const int b = row_ptr[r], e = row_ptr[r + 1];
    auto lower = [&](long long key) {
        int lo = b, hi = e;
        while (lo < hi) {
            int mid = lo + ((hi - lo) >> 1);
            if (col_idx[mid] < key) lo = mid + 1; else hi = mid;
        }
        return lo;
    };
    const int f0 = lower((long long)s * slab_cols);
    const int f1 = (s + 1 == num_slabs) ? e : lower((long long)(s + 1) * slab_cols);
    first[t] = f0;
    counts[t] = f1 - f0;
}

// Flags a row whose column ids decrease somewhere (tiling needs sorted rows).
__global__ __launch_bounds__(256) void tile_sorted_check_kernel(const int *__restrict__ row_ptr,
                                                                 const int *__restrict__ col_idx, int n_rows,
                                                                 int nnz, int *__restrict__ bad)
{
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e + 1 >= nnz) return;
    if (col_idx[e] <= col_idx[e + 1]) return;
    // a decrease is fine only where nonzero e + 1 starts a row
    int lo = 0, hi = n_rows;  // largest r with row_ptr[r] <= e + 1
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (row_ptr[mid] <= e + 1) lo = mid; else hi = mid - 1;
    }
    if (row_ptr[lo] != e + 1) atomicOr(bad, 1);
}

// One thread per nonzero: its place in the slab-major order.
__global__ __launch_bounds__(256) void tile_scatter_kernel(const int *__restrict__ row_ptr,
                                                            const int *__restrict__ col_idx, int n_rows, int nnz,
                                                            int num_slabs, int slab_cols,
                                                            const int *__restrict__ first,
                                                            const int *__restrict__ vrow_ptr,
                                                            int *__restrict__ col_tiled, int *__restrict__ perm)
{
    const long long e64 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e64 >= nnz) return;
    const int e = (int)e64;
    int lo = 0, hi = n_rows;  // largest r with row_ptr[r] <= e  (the row that holds nonzero e)
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (row_ptr[mid] <= e) lo = mid; else hi = mid - 1;
    }
    const int c = col_idx[e];
    int s = c / slab_cols;
    if (s >= num_slabs) s = num_slabs - 1;
    const long long v = (long long)s * n_rows + lo;
    const int dst = vrow_ptr[v] + (e - first[v]);
    col_tiled[dst] = c;
    perm[dst] = e;
}

// Y[r] = sum over slabs, in slab order, of the partial rows part[s * n_rows + r].
template <typename TOut, int VEC>
__global__ __launch_bounds__(256) void tile_reduce_kernel(const float *__restrict__ part, TOut *__restrict__ Y,
                                                           int n_rows, int K, int num_slabs)
{
    const size_t per_slab = (size_t)n_rows * K;
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (i >= per_slab) return;
    float acc[VEC];
#pragma unroll
    for (int u = 0; u < VEC; ++u) acc[u] = 0.f;
    for (int s = 0; s < num_slabs; ++s) {
        const float *p = part + (size_t)s * per_slab + i;
        if constexpr (VEC == 4) {
            float4 t = *reinterpret_cast<const float4 *>(p);
            acc[0] += t.x; acc[1] += t.y; acc[2] += t.z; acc[3] += t.w;
        } else {
            acc[0] += p[0];
        }
    }
    store_acc<VEC>(Y + i, acc);
}


// Rounds of wavefront w: the longest nonzero run among its partitions, in windows.
__global__ __launch_bounds__(256) void slice_count_kernel(const int *__restrict__ coord_y, int P, int tpw,
                                                           int num_waves, int *__restrict__ rounds)
{
    const int w = blockIdx.x * blockDim.x + threadIdx.x;
    if (w > num_waves) return;
    int r = 0;
    if (w < num_waves) {
        const int p0 = w * tpw;
        const int p1 = min(p0 + tpw, P);
        for (int p = p0; p < p1; ++p) r = max(r, (coord_y[p + 1] - coord_y[p] + kWindow - 1) / kWindow);
    }
    rounds[w] = r;
}

// One thread per (virtual-order) nonzero: its slot in the sliced arrays.
__global__ __launch_bounds__(256) void slice_scatter_kernel(const int *__restrict__ col_v,
                                                             const int *__restrict__ perm,
                                                             const int *__restrict__ coord_y, int P, int tpw,
                                                             const int *__restrict__ wave_off, int nnz,
                                                             int *__restrict__ slice_cols,
                                                             int *__restrict__ slice_src)
{
    const long long y64 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (y64 >= nnz) return;
    const int y = (int)y64;
    int lo = 0, hi = P - 1;  // largest p with coord_y[p] <= y
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (coord_y[mid] <= y) lo = mid; else hi = mid - 1;
    }
    const int p = lo;
    const int w = p / tpw, g = p - w * tpw;
    const int k = y - coord_y[p];
    const size_t slot = ((size_t)wave_off[w] + (size_t)(k / kWindow)) * (size_t)(tpw * kWindow) + (size_t)g * kWindow +
                        (size_t)(k % kWindow);
    slice_cols[slot] = col_v[y];
    slice_src[slot] = perm ? perm[y] : y;
}

template <typename T>
__global__ __launch_bounds__(256) void slice_values_kernel(const T *__restrict__ val,
                                                            const int *__restrict__ slice_src, size_t slots,
                                                            T *__restrict__ slice_vals)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= slots) return;
    const int src = slice_src[i];
    slice_vals[i] = src >= 0 ? val[src] : (T)0;
}

template <typename T>
int dev_alloc(mps_plan *pl, T **p, size_t count)
{
    size_t bytes = (count ? count : 1) * sizeof(T);
    MPS_HIP_TRY(hipMalloc(reinterpret_cast<void **>(p), bytes));
    pl->device_bytes += bytes;
    return MPS_OK;
}

void plan_free(mps_plan *pl)
{
    if (!pl) return;
    (void)hipFree(pl->vrow_ptr);
    (void)hipFree(pl->coord_x);
    (void)hipFree(pl->coord_y);
    (void)hipFree(pl->wave_off);
    (void)hipFree(pl->slice_cols);
    (void)hipFree(pl->slice_vals);
    (void)hipFree(pl->slice_src);
    (void)hipFree(pl->workspace);
    delete pl;
}

size_t part_bytes_for(int n_rows, int num_slabs, int K)
{
    if (num_slabs <= 1) return 0;
    size_t b = (size_t)num_slabs * (size_t)n_rows * K * sizeof(float);
    return (b + 255) / 256 * 256;
}

int plan_set_values(mps_plan *pl, const void *d_val, hipStream_t st)
{
    const size_t slots = (size_t)pl->total_rounds * (size_t)(pl->shape.tpw * kWindow);
    if (slots == 0) return MPS_OK;
    unsigned blocks = (unsigned)((slots + 255) / 256);
    if (pl->elem_bytes == 4)
        hipLaunchKernelGGL((slice_values_kernel<float>), dim3(blocks), dim3(256), 0, st,
                           static_cast<const float *>(d_val), pl->slice_src, slots,
                           static_cast<float *>(pl->slice_vals));
    else
        hipLaunchKernelGGL((slice_values_kernel<half_t>), dim3(blocks), dim3(256), 0, st,
                           static_cast<const half_t *>(d_val), pl->slice_src, slots,
                           static_cast<half_t *>(pl->slice_vals));
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

// Builds everything; temporaries are released before returning.
int plan_build(mps_plan *pl, const int *d_row_ptr, const int *d_col_idx, const void *d_val, unsigned flags,
               size_t slab_bytes, int tpw, hipStream_t st)
{
    const int n = pl->n_rows, nnz = pl->nnz, K = pl->K, eb = pl->elem_bytes;
    int rc;
    // 1. slabs
    pl->num_slabs = 1;
    pl->slab_cols = n > 0 ? n : 1;
    if (!(flags & MPS_PLAN_NO_TILING) && n > 0 && nnz > 0) {
        if (flags & MPS_PLAN_FORCE_TILING) {
            size_t sb = slab_bytes ? slab_bytes : kDefaultSlabBytes;
            long long cols = (long long)(sb / ((size_t)K * eb));
            cols = cols / 64 * 64;
            if (cols < 64) cols = 64;
            long long slabs = (n + cols - 1) / cols;
            if (slabs * n + 1 + nnz > INT_MAX) return MPS_ERR_UNSUPPORTED;
            pl->num_slabs = (int)slabs;
            pl->slab_cols = (int)cols;
        } else {
            rc = mps_tile_shape(n, nnz, K, eb, slab_bytes, &pl->num_slabs, &pl->slab_cols);
            if (rc != MPS_OK) return rc;
        }
    }
    int *first = nullptr, *col_v = nullptr, *perm = nullptr, *sums = nullptr;
    mps_plan tmp;  // byte accounting of temporaries is not kept
    auto drop_tmp = [&] {
        (void)hipFree(first);
        (void)hipFree(col_v);
        (void)hipFree(perm);
        (void)hipFree(sums);
        first = col_v = perm = sums = nullptr;
    };
    rc = dev_alloc(&tmp, &sums, (size_t)kScanMaxBlocks + 1);
    if (rc != MPS_OK) return rc;

    for (int attempt = 0; attempt < 2; ++attempt) {
        const long long nv = (long long)pl->num_slabs * n;
        pl->n_vrows = (int)nv;
        rc = dev_alloc(pl, &pl->vrow_ptr, (size_t)nv + 1);
        if (rc != MPS_OK) { drop_tmp(); return rc; }
        if (pl->num_slabs == 1) {
            MPS_HIP_TRY(hipMemcpyAsync(pl->vrow_ptr, d_row_ptr, ((size_t)n + 1) * sizeof(int),
                                       hipMemcpyDeviceToDevice, st));
            break;
        }
        // 2. slab-major order
        if ((rc = dev_alloc(&tmp, &first, (size_t)nv)) != MPS_OK || (rc = dev_alloc(&tmp, &col_v, (size_t)nnz)) != MPS_OK ||
            (rc = dev_alloc(&tmp, &perm, (size_t)nnz)) != MPS_OK) {
            drop_tmp();
            return rc;
        }
        int *bad = sums + kScanMaxBlocks;
        int zero = 0, h_bad = 0;
        MPS_HIP_TRY(hipMemcpyAsync(bad, &zero, sizeof(int), hipMemcpyHostToDevice, st));
        if (nnz > 1)
            hipLaunchKernelGGL(tile_sorted_check_kernel, dim3((unsigned)(((long long)nnz + 255) / 256)), dim3(256), 0, st,
                               d_row_ptr, d_col_idx, n, nnz, bad);
        hipLaunchKernelGGL(tile_count_kernel, dim3((unsigned)((nv + 1 + 255) / 256)), dim3(256), 0, st, d_row_ptr,
                           d_col_idx, n, pl->num_slabs, pl->slab_cols, first, pl->vrow_ptr);
        MPS_HIP_TRY(hipGetLastError());
        if ((rc = scan_exclusive_inplace(pl->vrow_ptr, (int)nv + 1, sums, st)) != MPS_OK) { drop_tmp(); return rc; }
        hipLaunchKernelGGL(tile_scatter_kernel, dim3((unsigned)(((long long)nnz + 255) / 256)), dim3(256), 0, st, d_row_ptr,
                           d_col_idx, n, nnz, pl->num_slabs, pl->slab_cols, first, pl->vrow_ptr, col_v, perm);
        MPS_HIP_TRY(hipGetLastError());
        MPS_HIP_TRY(hipMemcpyAsync(&h_bad, bad, sizeof(int), hipMemcpyDeviceToHost, st));
        MPS_HIP_TRY(hipStreamSynchronize(st));
        if (!h_bad) break;
        // rows are not sorted: tiling is impossible
        if (flags & MPS_PLAN_FORCE_TILING) { drop_tmp(); return MPS_ERR_UNSORTED; }
        (void)hipFree(first); (void)hipFree(col_v); (void)hipFree(perm);
        first = col_v = perm = nullptr;
        (void)hipFree(pl->vrow_ptr);
        pl->vrow_ptr = nullptr;
        pl->num_slabs = 1;
        pl->slab_cols = n;
    }
    const int *cols_v = pl->num_slabs == 1 ? d_col_idx : col_v;

    // 3. merge-path partition of the virtual rows
    if ((rc = mps_num_partitions(pl->n_vrows, nnz, pl->cost, &pl->P)) != MPS_OK) { drop_tmp(); return rc; }
    if ((rc = make_spmm_shape(n, K, pl->P, tpw, eb, pl->shape)) != MPS_OK) { drop_tmp(); return rc; }
    if ((rc = dev_alloc(pl, &pl->coord_x, (size_t)pl->P + 1)) != MPS_OK ||
        (rc = dev_alloc(pl, &pl->coord_y, (size_t)pl->P + 1)) != MPS_OK) { drop_tmp(); return rc; }
    if ((rc = mps_partition(pl->vrow_ptr, pl->n_vrows, nnz, pl->P, pl->coord_x, pl->coord_y, st)) != MPS_OK) {
        drop_tmp();
        return rc;
    }

    // 4. slices
    const int W = pl->shape.num_waves, G = pl->shape.tpw;
    if ((rc = dev_alloc(pl, &pl->wave_off, (size_t)W + 1)) != MPS_OK) { drop_tmp(); return rc; }
    hipLaunchKernelGGL(slice_count_kernel, dim3((unsigned)((W + 1 + 255) / 256)), dim3(256), 0, st, pl->coord_y, pl->P, G, W,
                       pl->wave_off);
    MPS_HIP_TRY(hipGetLastError());
    if ((rc = scan_exclusive_inplace(pl->wave_off, W + 1, sums, st)) != MPS_OK) { drop_tmp(); return rc; }
    int total_rounds = 0;
    MPS_HIP_TRY(hipMemcpyAsync(&total_rounds, pl->wave_off + W, sizeof(int), hipMemcpyDeviceToHost, st));
    MPS_HIP_TRY(hipStreamSynchronize(st));
    pl->total_rounds = total_rounds;
    const size_t slots = (size_t)total_rounds * (size_t)(G * kWindow);
    if ((rc = dev_alloc(pl, &pl->slice_cols, slots)) != MPS_OK || (rc = dev_alloc(pl, &pl->slice_src, slots)) != MPS_OK) {
        drop_tmp();
        return rc;
    }
    {
        unsigned char *sv = nullptr;
        if ((rc = dev_alloc(pl, &sv, (slots ? slots : 1) * (size_t)eb)) != MPS_OK) { drop_tmp(); return rc; }
        pl->slice_vals = sv;
    }
    if (slots) {
        MPS_HIP_TRY(hipMemsetAsync(pl->slice_cols, 0, slots * sizeof(int), st));
        MPS_HIP_TRY(hipMemsetAsync(pl->slice_src, 0xff, slots * sizeof(int), st));
    }
    if (nnz > 0) {
        hipLaunchKernelGGL(slice_scatter_kernel, dim3((unsigned)(((long long)nnz + 255) / 256)), dim3(256), 0, st, cols_v,
                           pl->num_slabs == 1 ? nullptr : perm, pl->coord_y, pl->P, G, pl->wave_off, nnz, pl->slice_cols,
                           pl->slice_src);
        MPS_HIP_TRY(hipGetLastError());
    }
    if ((rc = plan_set_values(pl, d_val, st)) != MPS_OK) { drop_tmp(); return rc; }

    // 5. workspace
    pl->part_bytes = part_bytes_for(n, pl->num_slabs, K);
    pl->workspace_bytes = pl->part_bytes + carry_bytes_for(W, K);
    {
        unsigned char *ws = nullptr;
        if ((rc = dev_alloc(pl, &ws, pl->workspace_bytes)) != MPS_OK) { drop_tmp(); return rc; }
        pl->workspace = ws;
    }
    MPS_HIP_TRY(hipStreamSynchronize(st));
    drop_tmp();
    return MPS_OK;
}

template <typename T>
int plan_spmm(const mps_plan *pl, const T *X, T *Y, unsigned phases, hipStream_t st)
{
    if (!pl || pl->elem_bytes != (int)sizeof(T)) return MPS_ERR_INVALID_ARG;
    if (pl->n_rows == 0) return MPS_OK;
    if (!X || !Y) return MPS_ERR_INVALID_ARG;
    if (!aligned_to(X, 16) || !aligned_to(Y, 16)) return MPS_ERR_ALIGNMENT;
    const T *vals = static_cast<const T *>(pl->slice_vals);
    void *carry = static_cast<char *>(pl->workspace) + pl->part_bytes;
    if (pl->num_slabs == 1)
        return launch_spmm_any<T, T>(pl->vrow_ptr, pl->slice_cols, vals, X, Y, pl->nnz, pl->K, pl->P, pl->coord_x,
                                     pl->coord_y, pl->wave_off, pl->shape, carry, phases, st);
    float *part = static_cast<float *>(pl->workspace);
    int rc = launch_spmm_any<T, float>(pl->vrow_ptr, pl->slice_cols, vals, X, part, pl->nnz, pl->K, pl->P, pl->coord_x,
                                       pl->coord_y, pl->wave_off, pl->shape, carry, phases, st);
    if (rc != MPS_OK) return rc;
    if (phases & MPS_PHASE_REDUCE) {
        const size_t per_slab = (size_t)pl->n_rows * pl->K;
        if (pl->K % 4 == 0)
            hipLaunchKernelGGL((tile_reduce_kernel<T, 4>), dim3((unsigned)((per_slab / 4 + 255) / 256)), dim3(256), 0, st,
                               part, Y, pl->n_rows, pl->K, pl->num_slabs);
        else
            hipLaunchKernelGGL((tile_reduce_kernel<T, 1>), dim3((unsigned)((per_slab + 255) / 256)), dim3(256), 0, st, part,
                               Y, pl->n_rows, pl->K, pl->num_slabs);
        MPS_HIP_TRY(hipGetLastError());
    }
    return MPS_OK;
}

}  // namespace

extern "C" {

int mps_tile_shape(int n_rows, int nnz, int K, int elem_bytes, size_t slab_bytes, int *num_slabs_out,
                   int *slab_cols_out)
{
    if (!num_slabs_out || !slab_cols_out || n_rows < 0 || nnz < 0 || K < 1) return MPS_ERR_INVALID_ARG;
    if (elem_bytes != 4 && elem_bytes != 2) return MPS_ERR_INVALID_ARG;
    if (slab_bytes == 0) slab_bytes = kDefaultSlabBytes;
    const uint64_t row_b = (uint64_t)K * elem_bytes;
    const uint64_t x_bytes = (uint64_t)n_rows * row_b;
    int slabs = 1, cols = n_rows > 0 ? n_rows : 1;
    // Worth it when X overflows one XCD's L2 (4 MiB) and the nonzeros of a row
    // inside one slab still form runs long enough to stream (>= 8 on average).
    if (x_bytes > (3u << 20) && n_rows > 0) {
        uint64_t want = (x_bytes + slab_bytes - 1) / slab_bytes;
        if (want > 4096) want = 4096;
        uint64_t per = ((uint64_t)n_rows + want - 1) / want;
        per = (per + 63) / 64 * 64;
        uint64_t s2 = ((uint64_t)n_rows + per - 1) / per;
        if ((double)nnz / ((double)n_rows * (double)s2) >= 8.0 &&
            (uint64_t)s2 * n_rows + 1 + (uint64_t)nnz <= (uint64_t)INT_MAX) {
            slabs = (int)s2;
            cols = (int)per;
        }
    }
    *num_slabs_out = slabs;
    *slab_cols_out = cols;
    return MPS_OK;
}

int mps_plan_create(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n_rows, int nnz, int K,
                    int elem_bytes, int cost, int tpw, unsigned flags, size_t slab_bytes, void *stream,
                    mps_plan **plan_out)
{
    if (!plan_out) return MPS_ERR_INVALID_ARG;
    *plan_out = nullptr;
    if (!d_row_ptr || n_rows < 0 || nnz < 0 || K < 1 || cost <= 0 || tpw < 0) return MPS_ERR_INVALID_ARG;
    if (elem_bytes != 4 && elem_bytes != 2) return MPS_ERR_INVALID_ARG;
    if (nnz > 0 && (!d_col_idx || !d_val)) return MPS_ERR_INVALID_ARG;
    if ((long long)n_rows + 1 + nnz > INT_MAX) return MPS_ERR_UNSUPPORTED;
    mps_plan *pl = new (std::nothrow) mps_plan;
    if (!pl) return MPS_ERR_INVALID_ARG;
    pl->n_rows = n_rows;
    pl->nnz = nnz;
    pl->K = K;
    pl->elem_bytes = elem_bytes;
    pl->cost = cost;
    int rc = plan_build(pl, d_row_ptr, d_col_idx, d_val, flags, slab_bytes, tpw, static_cast<hipStream_t>(stream));
    if (rc != MPS_OK) {
        plan_free(pl);
        return rc;
    }
    *plan_out = pl;
    return MPS_OK;
}

void mps_plan_destroy(mps_plan *plan) { plan_free(plan); }

int mps_plan_get_info(const mps_plan *plan, mps_plan_info *info)
{
    if (!plan || !info) return MPS_ERR_INVALID_ARG;
    info->n_rows = plan->n_rows;
    info->nnz = plan->nnz;
    info->K = plan->K;
    info->elem_bytes = plan->elem_bytes;
    info->cost = plan->cost;
    info->threads_per_wave = plan->shape.tpw;
    info->num_slabs = plan->num_slabs;
    info->slab_cols = plan->slab_cols;
    info->num_partitions = plan->P;
    info->num_waves = plan->shape.num_waves;
    info->total_rounds = plan->total_rounds;
    info->slice_slots = plan->total_rounds * (long long)(plan->shape.tpw * kWindow);
    info->device_bytes = plan->device_bytes;
    return MPS_OK;
}

int mps_plan_set_values(mps_plan *plan, const void *d_val, void *stream)
{
    if (!plan || (plan->nnz > 0 && !d_val)) return MPS_ERR_INVALID_ARG;
    return plan_set_values(plan, d_val, static_cast<hipStream_t>(stream));
}

int mps_plan_copy_array(const mps_plan *plan, int which, void *host_dst, size_t bytes)
{
    if (!plan || !host_dst) return MPS_ERR_INVALID_ARG;
    const void *src = nullptr;
    size_t have = 0;
    const size_t slots = (size_t)plan->total_rounds * (size_t)(plan->shape.tpw * kWindow);
    switch (which) {
    case MPS_PLAN_ARRAY_VROW_PTR: src = plan->vrow_ptr; have = ((size_t)plan->n_vrows + 1) * sizeof(int); break;
    case MPS_PLAN_ARRAY_COORD_X: src = plan->coord_x; have = ((size_t)plan->P + 1) * sizeof(int); break;
    case MPS_PLAN_ARRAY_COORD_Y: src = plan->coord_y; have = ((size_t)plan->P + 1) * sizeof(int); break;
    case MPS_PLAN_ARRAY_WAVE_OFF: src = plan->wave_off; have = ((size_t)plan->shape.num_waves + 1) * sizeof(int); break;
    case MPS_PLAN_ARRAY_SLICE_COLS: src = plan->slice_cols; have = slots * sizeof(int); break;
    case MPS_PLAN_ARRAY_SLICE_SRC: src = plan->slice_src; have = slots * sizeof(int); break;
    case MPS_PLAN_ARRAY_SLICE_VALS: src = plan->slice_vals; have = slots * (size_t)plan->elem_bytes; break;
    default: return MPS_ERR_INVALID_ARG;
    }
    if (bytes != have) return MPS_ERR_INVALID_ARG;
    if (have == 0) return MPS_OK;
    MPS_HIP_TRY(hipMemcpy(host_dst, src, have, hipMemcpyDeviceToHost));
    return MPS_OK;
}

int mps_plan_spmm_f32(const mps_plan *plan, const float *d_X, float *d_Y, void *stream)
{
    return plan_spmm<float>(plan, d_X, d_Y, MPS_PHASE_MAIN | MPS_PHASE_FIXUP | MPS_PHASE_REDUCE,
                            static_cast<hipStream_t>(stream));
}

int mps_plan_spmm_f16(const mps_plan *plan, const uint16_t *d_X, uint16_t *d_Y, void *stream)
{
    return plan_spmm<half_t>(plan, reinterpret_cast<const half_t *>(d_X), reinterpret_cast<half_t *>(d_Y),
                             MPS_PHASE_MAIN | MPS_PHASE_FIXUP | MPS_PHASE_REDUCE, static_cast<hipStream_t>(stream));
}

int mps_plan_spmm_phases(const mps_plan *plan, const void *d_X, void *d_Y, unsigned phases, void *stream)
{
    if (!plan) return MPS_ERR_INVALID_ARG;
    if (plan->elem_bytes == 4)
        return plan_spmm<float>(plan, static_cast<const float *>(d_X), static_cast<float *>(d_Y), phases,
                                static_cast<hipStream_t>(stream));
    return plan_spmm<half_t>(plan, static_cast<const half_t *>(d_X), static_cast<half_t *>(d_Y), phases,
                             static_cast<hipStream_t>(stream));
}

}  // extern "C"
