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
#include "mpspmm_rowblock.hpp"
#include "mpspmm_sweep.hpp"

#include <algorithm>
#include <cmath>
#include <new>
#include <vector>

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
    // hot columns (LDS-resident rows of X), tiled plans only
    int num_segs = 1;          // virtual-row segments: num_slabs, or 2 * num_slabs with hot columns
    int hot_rows = 0;          // rows of X per hot table (0: no hot launch)
    int hot_waves = 0;         // wavefronts [0, hot_waves) belong to hot segments
    long long hot_nnz = 0;     // nonzeros whose column is hot
    int *hot_cols = nullptr;   // [num_slabs][hot_rows] column ids by slot, -1 = unused
    int *seg_table = nullptr;  // [g] = first partition of hot segment g (g <= num_slabs)
    size_t hot_lds_bytes = 0;
    int hot_cost = 0;               // merge items per partition in the hot segments
    int mark_shift = 0, hot_mark_shift = 0;  // row marks sit above this bit of a column entry (0: none)
    bool streamed_flag = false;  // untiled plans: bit mark_shift of an entry marks a column outside the resident set
    bool column_tiles = false;   // untiled plans with wide rows of X: 8-lane groups, one pass per 128 bytes of row pitch
    int resident_cols = 0;       // columns whose rows of X are gathered without the streaming hint
    long long resident_nnz = 0;  // nonzeros in them
    int *hot_block_wave = nullptr;  // [hot_blocks + 1] first wave of every hot workgroup
    int hot_blocks = 0;
    bool keep_sources = true;       // slice_src is kept (mps_plan_set_values works)
    // degree weights (weights != 0): no value arrays; X is scaled by col_scale into xs before the kernels,
    // which add up rows of xs; finished rows are scaled by row_scale
    int weights = 0;                // 0: values from val; else 1 + MPS_WEIGHT_*
    float *col_scale = nullptr, *row_scale = nullptr;  // [n_rows] each
    float *xs = nullptr;            // [n_rows * K]
    mps_rb::DevicePlan *rb = nullptr;  // row-block plan: everything above about slabs and slices is unused
    mps_sw::DevicePlan *sw = nullptr;  // sweep plan: likewise
};

namespace {

// Slab of X that stays resident in a 4 MiB L2 next to the streamed data
// (3 MiB measured best on the power-law benchmark graph; 2 and 2.5 MiB within 5 %).
constexpr size_t kDefaultSlabBytes = 3u << 20;
constexpr size_t kDefaultResidentBytes = 10u << 20;  // rows of X that an untiled plan shields from streamed gathers
constexpr uint64_t kResidentMinXBytes = 192ull << 20;  // ... when X is this large
constexpr uint64_t kColumnTileMaxBytes = 160ull << 20;  // column tiles while one pass gathers from at most this much of X
constexpr double kResidentMinShare = 0.4;               // ... and the shielded columns hold this share of the nonzeros

// ---------------------------------------------------------------------------
// Cost model behind the automatic choices (slab size, hot columns), from
// measurements on MI355X with plans of power-law and uniform graphs of 0.2 to
// 2 M rows and 60 to 200 M nonzeros, K = 16 to 64.
//   * A gather costs one L1->L2 request per 128 bytes of a row of X, and the
//     time per request depends on how much of X the wavefronts that run
//     together spread their gathers over, and on how unevenly: with a 3 MiB
//     slab (the L2 of an XCD serves it) 5 ps whatever the matrix; with 12 MiB
//     6.8 ps on a power-law graph, whose popular columns stay in L2, and
//     11.7 ps on a uniform one; the tables below hold both ends.
//   * Skew is measured as the share of the nonzeros that lie in the busiest
//     tenth of the columns: 0.11 for a uniform graph, 0.54 to 0.65 for the
//     power-law graphs (exponent 2.1) measured, 0.41 and 0.31 for exponents
//     2.6 and 3.0; in between, the two tables are mixed (skew_from_share).  Unknown skew (negative): the power-law table, which
//     is the optimistic one for the untiled plan and so the cautious one for
//     tiling, and no slabs beyond 6 MiB.
//   * Every virtual row costs its fp32 partial row written once and read once:
//     2.8 ps per element of the row (45 ps at K = 16).
// ---------------------------------------------------------------------------
double request_ps(double table_bytes, double skew, bool tiled)
{
    // slabs of a tiled plan (measured at 3 .. 24 MiB) and the whole of X in an untiled one
    // (measured at 15 .. 128 MiB) are not the same curve: keep both
    static const double mib_t[] = {3, 6, 12, 24, 48, 96, 192, 384};
    static const double skewed_t[] = {5.3, 6.4, 6.8, 8.8, 11.7, 14.0, 16.0, 17.5};
    static const double uniform_t[] = {5.0, 6.9, 11.7, 15.0, 17.0, 18.5, 19.0, 19.5};
    static const double mib_u[] = {3, 6, 15, 32, 64, 128, 256, 512};
    static const double skewed_u[] = {5.3, 6.5, 9.4, 11.7, 14.0, 16.0, 17.5, 17.5};
    static const double uniform_u[] = {5.0, 6.9, 13.7, 16.5, 18.5, 19.0, 19.5, 19.5};
    const double *mib = tiled ? mib_t : mib_u, *skewed = tiled ? skewed_t : skewed_u, *uniform = tiled ? uniform_t : uniform_u;
    const double w = skew < 0 ? 1.0 : skew;
    const double m = table_bytes / (1024.0 * 1024.0);
    auto at = [&](int i) { return w * skewed[i] + (1.0 - w) * uniform[i]; };
    if (m <= mib[0]) return at(0);
    for (int i = 1; i < 8; ++i)
        if (m <= mib[i]) {
            const double t = std::log2(m / mib[i - 1]) / std::log2(mib[i] / mib[i - 1]);
            return at(i - 1) + t * (at(i) - at(i - 1));
        }
    return at(7);
}
constexpr double kPartialPsPerElement = 2.8;

// share of the nonzeros in the busiest tenth of the columns -> 0 (uniform) .. 1 (as skewed as the measured power-law graphs)
double skew_from_share(double top_tenth_share)
{
    // measured weights of the power-law table at 12 MiB slabs: share 0.63 -> 1, 0.59 -> 0.8, 0.41 -> 0.5, 0.31 -> 0.3, 0.11 -> 0
    const double s = (top_tenth_share - 0.11) / (0.63 - 0.11);
    return s <= 0 ? 0 : s >= 1 ? 1 : std::pow(s, 1.3);
}

// Modelled time (ps) of one product with X cut into slabs of slab_cols columns (num_slabs == 1: untiled).
double modelled_ps(int n_rows, int nnz, int K, int elem_bytes, int num_slabs, int slab_cols, double skew)
{
    const double row_bytes = (double)K * elem_bytes;
    const double requests = std::ceil(row_bytes / 128.0);
    const double table = (double)(num_slabs > 1 ? slab_cols : n_rows) * row_bytes;
    double t = (double)nnz * requests * request_ps(table, skew, num_slabs > 1);
    if (num_slabs > 1) t += (double)num_slabs * n_rows * K * kPartialPsPerElement;
    return t;
}

// The cheapest of {untiled, slabs of slab_bytes} or, with slab_bytes == 0, of
// {untiled, 3 MiB, 6 MiB} and, when the skew is known, {12 MiB, 24 MiB}.  A
// candidate must leave the rows of a slab runs long enough to stream (>= 4
// nonzeros per row and slab on average) and beat the untiled plan by 5 %.
void pick_tile_shape(int n_rows, int nnz, int K, int elem_bytes, size_t slab_bytes, double skew, int *num_slabs_out,
                     int *slab_cols_out)
{
    const uint64_t row_b = (uint64_t)K * elem_bytes;
    const uint64_t x_bytes = (uint64_t)n_rows * row_b;
    int slabs = 1, cols = n_rows > 0 ? n_rows : 1;
    size_t sizes[4] = {slab_bytes ? slab_bytes : kDefaultSlabBytes, 0, 0, 0};
    if (!slab_bytes) {
        sizes[1] = 2 * kDefaultSlabBytes;
        if (skew >= 0) {
            sizes[2] = 4 * kDefaultSlabBytes;
            sizes[3] = 8 * kDefaultSlabBytes;
        }
    }
    if (x_bytes > kDefaultSlabBytes && n_rows > 0) {
        double best = 0.95 * modelled_ps(n_rows, nnz, K, elem_bytes, 1, n_rows, skew);
        for (size_t sb : sizes) {
            if (sb == 0) continue;
            uint64_t want = (x_bytes + sb - 1) / sb;
            if (want < 2) continue;
            if (want > 4096) want = 4096;
            uint64_t per = ((uint64_t)n_rows + want - 1) / want;
            per = (per + 63) / 64 * 64;
            const uint64_t s2 = ((uint64_t)n_rows + per - 1) / per;
            if (s2 < 2 || (double)nnz / ((double)n_rows * (double)s2) < 4.0) continue;
            if (s2 * n_rows + 1 + (uint64_t)nnz > (uint64_t)INT_MAX) continue;
            const double t = modelled_ps(n_rows, nnz, K, elem_bytes, (int)s2, (int)per, skew);
            if (t < best) {
                best = t;
                slabs = (int)s2;
                cols = (int)per;
            }
        }
    }
    *num_slabs_out = slabs;
    *slab_cols_out = cols;
}

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
                                                            int *__restrict__ col_tiled, int *__restrict__ perm,
                                                            int *__restrict__ vrow_of)
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
    vrow_of[dst] = (int)v;
}

// Y[r] = sum over slabs, in slab order, of the partial rows part[s * n_rows + r].
template <typename TOut, int VEC>
__global__ __launch_bounds__(256) void tile_reduce_kernel(const float *__restrict__ part, TOut *__restrict__ Y,
                                                           int n_rows, int K, int num_slabs,
                                                           const float *__restrict__ row_scale)
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
    if (row_scale) {  // plans with degree weights: the row factor
        const float f = row_scale[i / (size_t)K];
#pragma unroll
        for (int u = 0; u < VEC; ++u) acc[u] *= f;
    }
    store_acc<VEC>(Y + i, acc);
}


// Degree weights as two factors per node: the weight of nonzero (r, c) is row_scale[r] * col_scale[c].
// Product mode: both the degree as a float (src/MergePathSpMM.cu:183-185, :450, :459 multiply them per
// nonzero).  GCN mode: 1 / sqrt(degree), 0 for an empty row.
__global__ __launch_bounds__(256) void degree_scales_kernel(const int *__restrict__ row_ptr, int n, int mode,
                                                             float *__restrict__ row_scale,
                                                             float *__restrict__ col_scale)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float d = (float)(row_ptr[i + 1] - row_ptr[i]);
    const float f = mode == MPS_WEIGHT_GCN ? (d > 0.f ? 1.0f / sqrtf(d) : 0.f) : d;
    row_scale[i] = f;
    col_scale[i] = f;
}

// xs[c][:] = col_scale[c] * X[c][:], four columns per thread (K % 4 == 0) or one.
template <int VEC>
__global__ __launch_bounds__(256) void scale_rows_kernel(const float *__restrict__ X,
                                                          const float *__restrict__ col_scale,
                                                          float *__restrict__ xs, int n, int K)
{
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (i >= (size_t)n * K) return;
    const float f = col_scale[i / (size_t)K];
    if constexpr (VEC == 4) {
        float4 t = *reinterpret_cast<const float4 *>(X + i);
        t.x *= f; t.y *= f; t.z *= f; t.w *= f;
        *reinterpret_cast<float4 *>(xs + i) = t;
    } else {
        xs[i] = f * X[i];
    }
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

// One thread per (virtual-order) nonzero: its slot in the sliced arrays.  With
// row marks (shift > 0: mark_shift for partitions from hot_parts on,
// hot_mark_shift before) the column entry also carries, above bit shift, the
// number of rows that end in front of this nonzero inside its partition: its
// virtual row minus that of the nonzero before it, or minus the row the
// partition starts in (coord_x - 1) for the partition's first nonzero.
// The virtual row of a nonzero comes from vrow_of (tiled plans: the scatter
// kernels know it) or from a bisection of vrow_ptr.  Its partition needs no
// search: the merge path passes through (row + 1, y) right before it consumes
// nonzero y, on diagonal row + 1 + y, and partition p owns the diagonals
// [p * ipt, (p + 1) * ipt) - of the whole matrix (seg == nullptr), or of the
// nonzero's segment (seg: seg_off[num_segs + 1], seg_parts[num_segs], seg_ipt[num_segs]).
// streamed (optional, int per column, 0 or 1): goes into bit shift of the entry, the row marks one bit higher.
__global__ __launch_bounds__(256) void slice_scatter_kernel(const int *__restrict__ col_v,
                                                             const int *__restrict__ perm,
                                                             const int *__restrict__ vrow_of,
                                                             const int *__restrict__ vrow_ptr, int n_vrows,
                                                             const int *__restrict__ coord_x,
                                                             const int *__restrict__ coord_y, int tpw,
                                                             const int *__restrict__ wave_off, int nnz, int ipt,
                                                             const int *__restrict__ seg, int num_segs, int seg_rows,
                                                             int hot_parts, int hot_mark_shift, int mark_shift,
                                                             const int *__restrict__ streamed,
                                                             int *__restrict__ slice_cols,
                                                             int *__restrict__ slice_src)
{
    const long long y64 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (y64 >= nnz) return;
    const int y = (int)y64;
    auto row_of = [&](int yy) {  // largest v with vrow_ptr[v] <= yy
        int a = 0, b = n_vrows - 1;
        while (a < b) {
            int mid = (a + b + 1) >> 1;
            if (vrow_ptr[mid] <= yy) a = mid; else b = mid - 1;
        }
        return a;
    };
    const int row = vrow_of ? vrow_of[y] : row_of(y);
    int p;
    if (seg) {
        const int g = row / seg_rows;
        const long long base = (long long)g * seg_rows;
        const long long d = (row - base) + 1 + (y - vrow_ptr[base]);
        p = seg[g] + (int)(d / seg[2 * num_segs + 1 + g]);
    } else {
        p = (int)(((long long)row + 1 + y) / ipt);
    }
    const int w = p / tpw, g = p - w * tpw;
    const int k = y - coord_y[p];
    const size_t slot = ((size_t)wave_off[w] + (size_t)(k / kWindow)) * (size_t)(tpw * kWindow) + (size_t)g * kWindow +
                        (size_t)(k % kWindow);
    unsigned entry = (unsigned)col_v[y];
    const int shift = p < hot_parts ? hot_mark_shift : mark_shift;
    if (shift > 0) {
        int before;
        if (k == 0) before = max(coord_x[p], 1) - 1;
        else if (vrow_of) before = vrow_of[y - 1];
        else before = vrow_ptr[row] < y ? row : row_of(y - 1);
        if (streamed) entry |= ((unsigned)streamed[col_v[y]] << shift) | ((unsigned)(row - before) << (shift + 1));
        else entry |= (unsigned)(row - before) << shift;
    }
    slice_cols[slot] = (int)entry;
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


// ---------------------------------------------------------------------------
// Hot columns.  Inside every column slab the hot_rows columns with the most
// nonzeros get their rows of X copied into LDS by the workgroups that process
// them ("hot" segments, gathered from LDS); the other columns of the slab form
// the "cold" segment, gathered through L2 as before.  Segment order: the hot
// segments of all slabs, then the cold segments; virtual row v = seg * n_rows + r.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void col_histogram_kernel(const int *__restrict__ col_idx, int nnz,
                                                             int *__restrict__ deg)
{
    const long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < nnz) atomicAdd(deg + col_idx[e], 1);
}

// Sixteen lanes per (slab, row): where the row's nonzeros of that slab start,
// and how many of them lie in hot columns.  (One thread per pair would walk a
// hub row's thousands of nonzeros alone while the rest of the launch waits.)
constexpr int kSplitLanes = 16;

__global__ __launch_bounds__(256) void hot_count_kernel(const int *__restrict__ row_ptr,
                                                         const int *__restrict__ col_idx, int n_rows,
                                                         int num_slabs, int slab_cols,
                                                         const int *__restrict__ hot_slot, int *__restrict__ first,
                                                         int *__restrict__ counts)
{
    const long long t = ((long long)blockIdx.x * blockDim.x + threadIdx.x) / kSplitLanes;
    const int sub = threadIdx.x & (kSplitLanes - 1);
    const long long nv = (long long)num_slabs * n_rows;
    if (t == nv && sub == 0) counts[2 * nv] = 0;
    if (t >= nv) return;  // whole 16-lane group
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
    int hot = 0;
    for (int i = f0 + sub; i < f1; i += kSplitLanes) hot += hot_slot[col_idx[i]] >= 0;
#pragma unroll
    for (int d = kSplitLanes / 2; d > 0; d >>= 1) hot += __shfl_xor(hot, d, kSplitLanes);
    if (sub == 0) {
        first[t] = f0;
        counts[t] = hot;                  // hot segment s
        counts[nv + t] = (f1 - f0) - hot; // cold segment num_slabs + s
    }
}

// Sixteen lanes per (slab, row): its nonzeros go, in order, to the hot or the
// cold virtual row; hot ones carry their LDS slot instead of the column id.
__global__ __launch_bounds__(256) void hot_scatter_kernel(const int *__restrict__ col_idx, int n_rows, int num_slabs,
                                                           const int *__restrict__ hot_slot,
                                                           const int *__restrict__ first,
                                                           const int *__restrict__ vrow_ptr,
                                                           int *__restrict__ col_out, int *__restrict__ perm,
                                                           int *__restrict__ vrow_of)
{
    const long long t = ((long long)blockIdx.x * blockDim.x + threadIdx.x) / kSplitLanes;
    const int lane = threadIdx.x & 63;
    const int sub = lane & (kSplitLanes - 1);
    const long long nv = (long long)num_slabs * n_rows;
    // lanes of a wavefront whose pair does not exist still take part in the ballots below
    const bool live = t < nv;
    int dh = 0, dc = 0, len = 0, f0 = 0;
    if (live) {
        dh = vrow_ptr[t];
        dc = vrow_ptr[nv + t];
        len = (vrow_ptr[t + 1] - dh) + (vrow_ptr[nv + t + 1] - dc);
        f0 = first[t];
    }
    int longest = len;  // the four groups of a wavefront loop together
#pragma unroll
    for (int d = 32; d >= kSplitLanes; d >>= 1) longest = max(longest, __shfl_xor(longest, d, 64));
    const int group_shift = lane & ~(kSplitLanes - 1);
    for (int base = 0; base < longest; base += kSplitLanes) {
        const int k = base + sub;
        const bool have = k < len;
        int c = 0, slot = -1;
        if (have) {
            c = col_idx[f0 + k];
            slot = hot_slot[c];
        }
        const unsigned long long hot_mask = __ballot(have && slot >= 0);
        const unsigned long long any_mask = __ballot(have);
        const unsigned mine_hot = (unsigned)(hot_mask >> group_shift) & 0xffffu;
        const unsigned mine_any = (unsigned)(any_mask >> group_shift) & 0xffffu;
        const unsigned below = (1u << sub) - 1u;
        if (have) {
            const int hot_before = __popc(mine_hot & below);
            if (slot >= 0) {
                col_out[dh + hot_before] = slot;
                perm[dh + hot_before] = f0 + k;
                vrow_of[dh + hot_before] = (int)t;
            } else {
                const int cold_before = __popc(mine_any & below) - hot_before;
                col_out[dc + cold_before] = c;
                perm[dc + cold_before] = f0 + k;
                vrow_of[dc + cold_before] = (int)(nv + t);
            }
        }
        const int nh = __popc(mine_hot);
        dh += nh;
        dc += __popc(mine_any) - nh;
    }
}

// Merge-path partition of every segment on its own (a partition never spans
// two segments, so a wavefront gathers either from LDS or from L2).  Thread i
// computes boundary i; seg_off[g] is the first partition of segment g,
// seg_parts[g] the number of its partitions that carry work (the rest, up to
// seg_off[g + 1], are empty padding), seg_ipt[g] its items per partition.
// The search is MergePathSearch (src/MergePathSpMM.cu:280-297) on the rows of
// the segment; x is returned as a global virtual-row coordinate.
__global__ __launch_bounds__(256) void seg_partition_kernel(const int *__restrict__ vrow_ptr, int n_rows,
                                                             int num_segs, const int *__restrict__ seg_off,
                                                             const int *__restrict__ seg_parts,
                                                             const int *__restrict__ seg_ipt, int P_total,
                                                             int *__restrict__ coord_x, int *__restrict__ coord_y)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i > P_total) return;
    int lo = 0, hi = num_segs - 1;  // largest g with seg_off[g] <= i
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (seg_off[mid] <= i) lo = mid; else hi = mid - 1;
    }
    const int g = lo;
    const int li = i - seg_off[g];
    const long long base = (long long)g * n_rows;
    const int y0 = vrow_ptr[base];
    const int nnz_g = vrow_ptr[base + n_rows] - y0;
    const int num_rows = n_rows + 1;
    const int total = num_rows + nnz_g;
    long long d64 = (long long)seg_ipt[g] * li;
    int diagonal = (li <= seg_parts[g] && d64 < (long long)total) ? (int)d64 : total;
    int x_min = max(diagonal - nnz_g, 0);
    int x_max = min(diagonal, num_rows);
    while (x_min < x_max) {
        int pivot = (x_min + x_max) >> 1;
        if (vrow_ptr[base + pivot] - y0 <= diagonal - pivot - 1)
            x_min = pivot + 1;
        else
            x_max = pivot;
    }
    const int x_l = min(x_min, num_rows);
    coord_x[i] = (int)base + max(x_l, 1);  // row base + x_l - 1 is in progress; a segment starts with its row 0
    coord_y[i] = y0 + (diagonal - x_min);
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
    mps_rb::destroy(pl->rb);
    mps_sw::destroy(pl->sw);
    (void)hipFree(pl->vrow_ptr);
    (void)hipFree(pl->coord_x);
    (void)hipFree(pl->coord_y);
    (void)hipFree(pl->wave_off);
    (void)hipFree(pl->slice_cols);
    (void)hipFree(pl->slice_vals);
    (void)hipFree(pl->slice_src);
    (void)hipFree(pl->workspace);
    (void)hipFree(pl->hot_cols);
    (void)hipFree(pl->seg_table);
    (void)hipFree(pl->hot_block_wave);
    (void)hipFree(pl->col_scale);
    (void)hipFree(pl->row_scale);
    (void)hipFree(pl->xs);
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

// Static LDS of a hot workgroup (see mp_spmm_kernel) and the rows of X that
// fit beside it in the 160 KiB of a CU.
constexpr int kHotCost = 256;  // most merge items per partition of a hot segment (unless the plan's cost is larger)

size_t hot_static_lds(int vec)
{
    const size_t comb = 64 * (size_t)vec;
    const size_t stage = comb > 2 * 16 * kWindow ? comb : 2 * 16 * kWindow;
    return kHotWavesPerBlock * (stage + comb) * sizeof(float) + kHotWavesPerBlock * 16 * sizeof(int);
}

int choose_hot_rows(int K, int eb, const SpmmShape &sh, bool force)
{
    if (sh.row_shift < 0 || sh.ls.vec == 1 || sh.ls.col_tiles != 1) return 0;
    // Measured on MI355X (Chung-Lu 233k): with 64-byte rows of X the hot launch wins
    // (0.58 against 0.66 ms at K = 16 fp32); with 128-byte rows and more the L2 path
    // moves twice the bytes per request at no extra cost while the LDS table holds
    // half the rows, and the hot launch loses (1.16 against 0.99 ms at K = 32).
    // fp16 rows of 64 bytes (K = 32): 8 conversions and 8 multiply-adds per lane and nonzero make the
    // hot launch ALU-bound; it runs as fast as the L2 path and costs a second set of partial rows
    // (0.672 ms either way), so it is not used.  fp16 rows of 32 bytes (K = 16) have half the
    // arithmetic per lane and twice the rows in the table: 0.555 against 0.659 ms.
    if (!force && (size_t)K * eb > (eb == 4 ? 64u : 32u)) return 0;
    const size_t budget = 160 * 1024 - hot_static_lds(sh.ls.vec) - 2048;
    size_t rows = budget / ((size_t)K * eb);
    rows = rows / 64 * 64;
    return rows >= 256 ? (int)rows : 0;
}

struct BuildTmp {
    int *first = nullptr, *col_v = nullptr, *perm = nullptr, *vrow = nullptr, *sums = nullptr, *deg = nullptr,
        *hot_slot = nullptr, *seg = nullptr;
    void drop()
    {
        (void)hipFree(first);
        (void)hipFree(col_v);
        (void)hipFree(perm);
        (void)hipFree(vrow);
        (void)hipFree(sums);
        (void)hipFree(deg);
        (void)hipFree(hot_slot);
        (void)hipFree(seg);
        first = col_v = perm = vrow = sums = deg = hot_slot = seg = nullptr;
    }
    ~BuildTmp() { drop(); }
};

template <typename T>
int tmp_alloc(T **p, size_t count)
{
    MPS_HIP_TRY(hipMalloc(reinterpret_cast<void **>(p), (count ? count : 1) * sizeof(T)));
    return MPS_OK;
}

// Picks the hot columns of every slab (host side, from the column histogram):
// the hot_rows columns with the most nonzeros, ties to the smaller column id;
// slots are handed out in ascending column order.  Returns the number of
// nonzeros that fall into hot columns.
long long select_hot_columns(const std::vector<int> &deg, int n, int num_slabs, int slab_cols, int hot_rows,
                             std::vector<int> &hot_slot, std::vector<int> &hot_cols)
{
    hot_slot.assign((size_t)n, -1);
    hot_cols.assign((size_t)num_slabs * hot_rows, -1);
    long long hot_nnz = 0;
    std::vector<int> order;
    for (int s = 0; s < num_slabs; ++s) {
        const int c0 = (int)std::min<long long>((long long)s * slab_cols, n);
        const int c1 = (int)std::min<long long>((long long)(s + 1) * slab_cols, n);
        order.resize((size_t)(c1 - c0));
        for (int c = c0; c < c1; ++c) order[(size_t)(c - c0)] = c;
        const size_t take = std::min<size_t>((size_t)hot_rows, order.size());
        auto hotter = [&](int a, int b) { return deg[a] != deg[b] ? deg[a] > deg[b] : a < b; };
        if (take < order.size()) std::nth_element(order.begin(), order.begin() + (long)take, order.end(), hotter);
        std::sort(order.begin(), order.begin() + (long)take);
        int slot = 0;
        for (size_t k = 0; k < take; ++k) {
            const int c = order[k];
            if (deg[c] == 0) continue;  // a column nobody references needs no slot
            hot_slot[(size_t)c] = slot;
            hot_cols[(size_t)s * hot_rows + slot] = c;
            hot_nnz += deg[c];
            ++slot;
        }
    }
    return hot_nnz;
}

// Builds everything; temporaries are released before returning.
int plan_build(mps_plan *pl, const int *d_row_ptr, const int *d_col_idx, const void *d_val, unsigned flags,
               size_t slab_bytes, size_t resident_bytes, int tpw, hipStream_t st)
{
    const int n = pl->n_rows, nnz = pl->nnz, K = pl->K, eb = pl->elem_bytes;
    int rc;
    // The histogram, the hot-column tables and the row marks all index by column id: a column
    // beyond the matrix (it is square) would write out of bounds or corrupt the marks.
    if ((rc = mps_csr_validate(d_row_ptr, d_col_idx, n, n, nnz, st)) != MPS_OK) return rc;
    // lane shape and partitions per wavefront do not depend on the partition count
    if ((rc = make_spmm_shape(n, K, 1, tpw, eb, pl->shape)) != MPS_OK) return rc;
    int G = pl->shape.tpw;

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
            pick_tile_shape(n, nnz, K, eb, slab_bytes, -1.0, &pl->num_slabs, &pl->slab_cols);
        }
    }
    BuildTmp t;
    if ((rc = tmp_alloc(&t.sums, (size_t)kScanMaxBlocks + 1)) != MPS_OK) return rc;
#define MPS_BUILD_TRY(expr)                       \
    do {                                          \
        int rc_ = (expr);                         \
        if (rc_ != MPS_OK) {                      \
            t.drop();                             \
            return rc_;                           \
        }                                         \
    } while (0)
#define MPS_BUILD_HIP(expr)                                     \
    do {                                                        \
        hipError_t e_ = (expr);                                 \
        if (e_ != hipSuccess) {                                 \
            t.drop();                                           \
            return MPS_ERR_HIP + (int)e_;                       \
        }                                                       \
    } while (0)

    // Nonzeros per column, on the host (once, for whoever needs it below).
    std::vector<int> h_deg;
    auto column_histogram = [&]() -> int {
        if (!h_deg.empty()) return MPS_OK;
        h_deg.resize((size_t)n);
        MPS_BUILD_TRY(tmp_alloc(&t.deg, (size_t)n));
        MPS_BUILD_HIP(hipMemsetAsync(t.deg, 0, (size_t)n * sizeof(int), st));
        hipLaunchKernelGGL(col_histogram_kernel, dim3((unsigned)(((long long)nnz + 255) / 256)), dim3(256), 0, st, d_col_idx,
                           nnz, t.deg);
        MPS_BUILD_HIP(hipGetLastError());
        MPS_BUILD_HIP(hipMemcpyAsync(h_deg.data(), t.deg, (size_t)n * sizeof(int), hipMemcpyDeviceToHost, st));
        MPS_BUILD_HIP(hipStreamSynchronize(st));
        return MPS_OK;
    };

    // 1b. Slabs of 12 and 24 MiB pay on skewed matrices only: where X is large enough for them
    // to matter, measure the skew (share of the nonzeros in the busiest tenth of the columns)
    // and choose again.
    if (!(flags & (MPS_PLAN_NO_TILING | MPS_PLAN_FORCE_TILING)) && slab_bytes == 0 && n >= 10 &&
        (uint64_t)n * K * eb > 8 * kDefaultSlabBytes && (long long)nnz >= 16LL * n) {
        MPS_BUILD_TRY(column_histogram());
        std::vector<int> d(h_deg);
        const size_t tenth = d.size() / 10;
        std::nth_element(d.begin(), d.begin() + (long)tenth, d.end(), [](int a, int b) { return a > b; });
        long long top = 0;
        for (size_t i = 0; i < tenth; ++i) top += d[i];
        pick_tile_shape(n, nnz, K, eb, 0, skew_from_share((double)top / (double)nnz), &pl->num_slabs, &pl->slab_cols);
    }

    // 2. hot columns of every slab (tiled plans, shapes the hot kernel supports)
    int hot_rows = 0;
    std::vector<int> h_hot_cols;
    if (pl->num_slabs > 1 && !(flags & MPS_PLAN_NO_HOT)) {
        hot_rows = choose_hot_rows(K, eb, pl->shape, (flags & MPS_PLAN_FORCE_HOT) != 0);
        // Slabs beyond the L2 live on the hits of their popular columns; taking exactly those
        // columns out leaves the cold launch with the misses (500,000-row power-law graph,
        // 3 slabs of 10 MiB: 0.81 ms with hot columns, 0.79 ms without).
        if (!(flags & MPS_PLAN_FORCE_HOT) && (uint64_t)pl->slab_cols * K * eb > (4u << 20)) hot_rows = 0;
        if (2LL * pl->num_slabs * n + 1 + nnz > INT_MAX) hot_rows = 0;
        if (hot_rows > 0) {
            std::vector<int> h_slot;
            MPS_BUILD_TRY(column_histogram());
            pl->hot_nnz = select_hot_columns(h_deg, n, pl->num_slabs, pl->slab_cols, hot_rows, h_slot, h_hot_cols);
            // Worth a second launch and twice the partial rows?  Measured on MI355X at 64-byte rows,
            // graphs of 0.1 to 0.5 M rows with 3 to 45 M nonzeros in hot columns: a gather from LDS
            // saves 2.7 ps against one through L2; the second launch costs 15 us whatever its size
            // (table fill, tail, more carry records); a virtual row of the hot segments costs 1.7 ps
            // per element while the partial rows of the plan fit the 256 MiB last-level cache and
            // 4 ps per element once they do not.
            const double vrows = (double)pl->num_slabs * n;
            const double partial_bytes = 2.0 * vrows * K * sizeof(float);
            const double gain_ps = 2.7 * (double)pl->hot_nnz - vrows * K * (partial_bytes > 256.0 * 1048576.0 ? 4.0 : 1.7) - 15e6;
            if (gain_ps <= 0 && !(flags & MPS_PLAN_FORCE_HOT)) {
                hot_rows = 0;
                pl->hot_nnz = 0;
            } else {
                MPS_BUILD_TRY(tmp_alloc(&t.hot_slot, (size_t)n));
                MPS_BUILD_HIP(hipMemcpyAsync(t.hot_slot, h_slot.data(), (size_t)n * sizeof(int), hipMemcpyHostToDevice, st));
                MPS_BUILD_HIP(hipStreamSynchronize(st));
            }
        }
    }

    // 3. slab-major (and hot-first) order of the nonzeros
    for (int attempt = 0; attempt < 2; ++attempt) {
        pl->num_segs = pl->num_slabs * (hot_rows > 0 ? 2 : 1);
        const long long nslab_rows = (long long)pl->num_slabs * n;
        const long long nv = (long long)pl->num_segs * n;
        pl->n_vrows = (int)nv;
        MPS_BUILD_TRY(dev_alloc(pl, &pl->vrow_ptr, (size_t)nv + 1));
        if (pl->num_slabs == 1) {
            MPS_BUILD_HIP(hipMemcpyAsync(pl->vrow_ptr, d_row_ptr, ((size_t)n + 1) * sizeof(int), hipMemcpyDeviceToDevice, st));
            break;
        }
        MPS_BUILD_TRY(tmp_alloc(&t.first, (size_t)nslab_rows));
        MPS_BUILD_TRY(tmp_alloc(&t.col_v, (size_t)nnz));
        MPS_BUILD_TRY(tmp_alloc(&t.perm, (size_t)nnz));
        MPS_BUILD_TRY(tmp_alloc(&t.vrow, (size_t)nnz));
        int *bad = t.sums + kScanMaxBlocks;
        int zero = 0, h_bad = 0;
        MPS_BUILD_HIP(hipMemcpyAsync(bad, &zero, sizeof(int), hipMemcpyHostToDevice, st));
        if (nnz > 1)
            hipLaunchKernelGGL(tile_sorted_check_kernel, dim3((unsigned)(((long long)nnz + 255) / 256)), dim3(256), 0, st,
                               d_row_ptr, d_col_idx, n, nnz, bad);
        MPS_BUILD_HIP(hipMemcpyAsync(&h_bad, bad, sizeof(int), hipMemcpyDeviceToHost, st));
        MPS_BUILD_HIP(hipStreamSynchronize(st));
        if (h_bad) {
            // rows are not sorted: tiling is impossible
            if (flags & MPS_PLAN_FORCE_TILING) {
                t.drop();
                return MPS_ERR_UNSORTED;
            }
            (void)hipFree(t.first); (void)hipFree(t.col_v); (void)hipFree(t.perm); (void)hipFree(t.vrow);
            t.first = t.col_v = t.perm = t.vrow = nullptr;
            (void)hipFree(pl->vrow_ptr);
            pl->vrow_ptr = nullptr;
            pl->num_slabs = 1;
            pl->slab_cols = n;
            hot_rows = 0;
            pl->hot_nnz = 0;
            continue;
        }
        const unsigned row_blocks = (unsigned)((nslab_rows + 1 + 255) / 256);
        if (hot_rows > 0) {
            const unsigned split_blocks = (unsigned)(((nslab_rows + 1) * kSplitLanes + 255) / 256);
            hipLaunchKernelGGL(hot_count_kernel, dim3(split_blocks), dim3(256), 0, st, d_row_ptr, d_col_idx, n, pl->num_slabs,
                               pl->slab_cols, t.hot_slot, t.first, pl->vrow_ptr);
            MPS_BUILD_HIP(hipGetLastError());
            MPS_BUILD_TRY(scan_exclusive_inplace(pl->vrow_ptr, (int)nv + 1, t.sums, st));
            hipLaunchKernelGGL(hot_scatter_kernel, dim3(split_blocks), dim3(256), 0, st, d_col_idx, n, pl->num_slabs,
                               t.hot_slot, t.first, pl->vrow_ptr, t.col_v, t.perm, t.vrow);
        } else {
            hipLaunchKernelGGL(tile_count_kernel, dim3(row_blocks), dim3(256), 0, st, d_row_ptr, d_col_idx, n, pl->num_slabs,
                               pl->slab_cols, t.first, pl->vrow_ptr);
            MPS_BUILD_HIP(hipGetLastError());
            MPS_BUILD_TRY(scan_exclusive_inplace(pl->vrow_ptr, (int)nv + 1, t.sums, st));
            hipLaunchKernelGGL(tile_scatter_kernel, dim3((unsigned)(((long long)nnz + 255) / 256)), dim3(256), 0, st,
                               d_row_ptr, d_col_idx, n, nnz, pl->num_slabs, pl->slab_cols, t.first, pl->vrow_ptr, t.col_v,
                               t.perm, t.vrow);
        }
        MPS_BUILD_HIP(hipGetLastError());
        break;
    }
    const int *cols_v = pl->num_slabs == 1 ? d_col_idx : t.col_v;
    pl->hot_rows = hot_rows;

    // 3b. Column tiles for wide rows of X (untiled plans, short matrix rows, the caller left the partitions per
    // wavefront to the library).  A lane-group of 8 lanes covers 128 bytes of a row of X and the launch passes over
    // the matrix once per 128 bytes of row pitch (blockIdx.y), so that one pass gathers from N * 128 bytes instead
    // of the whole X, which the 256 MiB last-level cache then holds.  Measured on MI355X, R-MAT with 1 M rows and
    // 16 nonzeros per row: K = 256 2.07 against 2.34 ms (full rows, with resident columns), K = 128 0.98 against
    // 1.01 ms; K = 64 loses (0.51 against 0.49 ms) and keeps full rows.  The sparse arrays are read once per pass:
    // with long matrix rows they are the larger part of the traffic, so those keep full rows too.  The merge items
    // per wavefront stay what the caller's cost gave them.
    if (tpw == 0 && pl->num_slabs == 1 && hot_rows == 0 && !(flags & MPS_PLAN_NO_COLUMN_TILES) && !pl->weights &&
        pl->shape.ls.vec * eb == 16 && (uint64_t)K * eb >= 512 && ((uint64_t)K * eb) % 128 == 0 &&
        (long long)nnz < 64LL * n && (uint64_t)n * 128 <= kColumnTileMaxBytes) {
        const int old_groups = pl->shape.ls.groups;
        pl->shape.ls.lanes_log2 = 3;
        pl->shape.ls.groups = 8;
        pl->shape.ls.col_tiles = (int)(((uint64_t)K * eb) / 128);
        pl->shape.tpw = G = 8;
        long long c = (long long)pl->cost * old_groups / 8;
        pl->cost = (int)(c < 16 ? 16 : c);
        pl->column_tiles = true;
    }

    // 4. merge-path partition of the virtual rows
    int max_cold_ipt = 0, max_hot_ipt = 0;
    if (hot_rows == 0) {
        // one split of all virtual rows: the reference's (src/MergePathSpMM.cu:138-139, :327-334)
        MPS_BUILD_TRY(mps_num_partitions(pl->n_vrows, nnz, pl->cost, &pl->P));
        MPS_BUILD_TRY(dev_alloc(pl, &pl->coord_x, (size_t)pl->P + 1));
        MPS_BUILD_TRY(dev_alloc(pl, &pl->coord_y, (size_t)pl->P + 1));
        MPS_BUILD_TRY(mps_partition(pl->vrow_ptr, pl->n_vrows, nnz, pl->P, pl->coord_x, pl->coord_y, st));
        pl->hot_waves = 0;
        MPS_BUILD_TRY(mps_items_per_partition(pl->n_vrows, nnz, pl->P, &max_cold_ipt));
    } else {
        // every segment is split on its own and padded to whole wavefronts
        const int S2 = pl->num_segs, S = pl->num_slabs;
        std::vector<int> seg_y((size_t)S2 + 1);
        for (int g = 0; g <= S2; ++g)
            MPS_BUILD_HIP(hipMemcpyAsync(&seg_y[(size_t)g], pl->vrow_ptr + (size_t)g * n, sizeof(int), hipMemcpyDeviceToHost, st));
        MPS_BUILD_HIP(hipStreamSynchronize(st));
        {
            // Hot segments take long partitions (nothing to gain from small ones where every
            // gather costs the same, and a long one hides the start-up loads), but every one
            // of the 16 wavefronts of the 256 hot workgroups should get a piece: measured on a
            // 100,000-row graph with 7.4 M hot nonzeros, cost 256 leaves 9 of 16 wavefronts
            // idle (0.169 ms per product), cost 128 runs at 0.146 ms.
            const long long hot_items = (long long)S * (n + 1) + (seg_y[(size_t)S] - seg_y[0]);
            long long fit = hot_items / (16LL * kHotWavesPerBlock * 256);
            if (fit > kHotCost) fit = kHotCost;
            if (fit < 64) fit = 64;
            pl->hot_cost = pl->cost > (int)fit ? pl->cost : (int)fit;
        }
        std::vector<int> h_seg((size_t)3 * S2 + 1);  // seg_off[S2 + 1], seg_parts[S2], seg_ipt[S2]
        int *seg_off = h_seg.data(), *seg_parts = seg_off + S2 + 1, *seg_ipt = seg_parts + S2;
        long long off = 0;
        for (int g = 0; g < S2; ++g) {
            const long long total = (long long)n + 1 + (seg_y[(size_t)g + 1] - seg_y[(size_t)g]);
            long long parts = (total - 1) / (g < S ? pl->hot_cost : pl->cost);
            if (parts < 1) parts = 1;
            const long long mult = G;  // whole wavefronts
            seg_off[g] = (int)off;
            seg_parts[g] = (int)parts;
            seg_ipt[g] = (int)((total + parts - 1) / parts);
            int &worst = g < S ? max_hot_ipt : max_cold_ipt;
            if (seg_ipt[g] > worst) worst = seg_ipt[g];
            off += (parts + mult - 1) / mult * mult;
            if (off > INT_MAX / 2) {
                t.drop();
                return MPS_ERR_UNSUPPORTED;
            }
        }
        seg_off[S2] = (int)off;
        pl->P = (int)off;
        pl->hot_waves = seg_off[S] / G;
        MPS_BUILD_TRY(tmp_alloc(&t.seg, h_seg.size()));
        MPS_BUILD_HIP(hipMemcpyAsync(t.seg, h_seg.data(), h_seg.size() * sizeof(int), hipMemcpyHostToDevice, st));
        MPS_BUILD_TRY(dev_alloc(pl, &pl->coord_x, (size_t)pl->P + 1));
        MPS_BUILD_TRY(dev_alloc(pl, &pl->coord_y, (size_t)pl->P + 1));
        hipLaunchKernelGGL(seg_partition_kernel, dim3((unsigned)(((long long)pl->P + 1 + 255) / 256)), dim3(256), 0, st,
                           pl->vrow_ptr, n, S2, t.seg, t.seg + S2 + 1, t.seg + 2 * S2 + 1, pl->P, pl->coord_x, pl->coord_y);
        MPS_BUILD_HIP(hipGetLastError());
        // what the hot kernel needs: slot -> column lists, and where the hot segments start
        std::vector<int> h_table((size_t)S + 1);
        for (int g = 0; g <= S; ++g) h_table[(size_t)g] = seg_off[g];
        MPS_BUILD_TRY(dev_alloc(pl, &pl->seg_table, h_table.size()));
        MPS_BUILD_HIP(hipMemcpyAsync(pl->seg_table, h_table.data(), h_table.size() * sizeof(int), hipMemcpyHostToDevice, st));
        MPS_BUILD_TRY(dev_alloc(pl, &pl->hot_cols, h_hot_cols.size()));
        MPS_BUILD_HIP(hipMemcpyAsync(pl->hot_cols, h_hot_cols.data(), h_hot_cols.size() * sizeof(int), hipMemcpyHostToDevice, st));
        MPS_BUILD_HIP(hipStreamSynchronize(st));
        pl->hot_lds_bytes = (size_t)hot_rows * K * eb;
        // the hot launch's dynamic LDS limit, once (not at every product): tiled plans write fp32 partial rows
        const int lds_rc = eb == 4 ? (allow_hot_lds<float, float>(pl->shape, pl->hot_lds_bytes))
                                   : (allow_hot_lds<half_t, float>(pl->shape, pl->hot_lds_bytes));
        MPS_BUILD_TRY(lds_rc);
        // Hot workgroups: one LDS table per CU at a time, so a few long-lived
        // workgroups per CU, each with a contiguous share of one segment's waves.
        int dev = 0, cus = 256;
        MPS_BUILD_HIP(hipGetDevice(&dev));
        MPS_BUILD_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        const long long target = cus;
        // Workgroups per segment in proportion to its wavefronts, never more than `target` in
        // all: one workgroup too many would run alone after all the others (6 segments at 43
        // workgroups each on 256 CUs took 0.66 instead of 0.55 ms).  Largest remainders first.
        std::vector<long long> seg_blocks((size_t)S), seg_rest((size_t)S);
        long long given = 0;
        const long long all_waves = pl->hot_waves > 0 ? pl->hot_waves : 1;
        for (int g = 0; g < S; ++g) {
            const long long wg = seg_off[g + 1] / G - seg_off[g] / G;
            seg_blocks[(size_t)g] = target * wg / all_waves;
            seg_rest[(size_t)g] = target * wg % all_waves;
            if (seg_blocks[(size_t)g] < 1) {
                seg_blocks[(size_t)g] = 1;
                seg_rest[(size_t)g] = 0;
            }
            given += seg_blocks[(size_t)g];
        }
        while (given < target) {
            int best = -1;
            for (int g = 0; g < S; ++g)
                if (seg_rest[(size_t)g] > 0 && (best < 0 || seg_rest[(size_t)g] > seg_rest[(size_t)best])) best = g;
            if (best < 0) break;
            ++seg_blocks[(size_t)best];
            seg_rest[(size_t)best] = 0;
            ++given;
        }
        std::vector<int> h_blocks;
        for (int g = 0; g < S; ++g) {
            const int w0 = seg_off[g] / G, w1 = seg_off[g + 1] / G;
            const long long wg = w1 - w0;
            long long blocks = seg_blocks[(size_t)g];
            const long long most = (wg + kHotWavesPerBlock - 1) / kHotWavesPerBlock;
            if (blocks > most) blocks = most;
            if (blocks < 1) blocks = 1;
            // equal shares, whatever the remainder: the 16 wavefronts of a workgroup
            // take the pieces of its share in turn
            for (long long b = 0; b < blocks; ++b) h_blocks.push_back((int)(w0 + wg * b / blocks));
        }
        h_blocks.push_back(pl->hot_waves);
        pl->hot_blocks = (int)h_blocks.size() - 1;
        MPS_BUILD_TRY(dev_alloc(pl, &pl->hot_block_wave, h_blocks.size()));
        MPS_BUILD_HIP(hipMemcpyAsync(pl->hot_block_wave, h_blocks.data(), h_blocks.size() * sizeof(int), hipMemcpyHostToDevice, st));
        MPS_BUILD_HIP(hipStreamSynchronize(st));
    }
    pl->shape.num_waves = (pl->P + G - 1) / G;
    // Row marks: a partition holds at most items-per-partition row ends, so that
    // many values must fit above the column (or LDS slot) bits of an entry.
    auto bits_for = [](long long v) { int b = 1; while ((v >> b) != 0) ++b; return b; };  // values 0..v
    {
        const int col_bits = bits_for(n > 1 ? n - 1 : 1);
        pl->mark_shift = (!(flags & MPS_PLAN_NO_ROW_MARKS) && nnz > 0 && col_bits + bits_for(max_cold_ipt) <= 32) ? col_bits : 0;
        if (hot_rows > 0) {
            const int slot_bits = bits_for(hot_rows - 1);
            if (slot_bits + bits_for(max_hot_ipt) > 32) {
                t.drop();
                return MPS_ERR_UNSUPPORTED;
            }
            pl->hot_mark_shift = slot_bits;
        }
        // Resident columns (untiled plans): the columns with the most nonzeros, as many as fit
        // resident_bytes, are gathered as usual; the entries of all other columns carry a flag and are
        // gathered with the streaming hint, so that the popular rows of X outlive in the caches the rows
        // that are used once or twice.  Measured on MI355X (R-MAT, 16 nonzeros per row, 1 and 4 M rows):
        // the hint makes a gather that misses dearer, so it pays only where the resident columns hold a
        // good share of the nonzeros and X is beyond the 256 MiB last-level cache: X of 256 MiB to 1 GiB
        // with 8 to 12 MiB resident (47 to 73 % of the nonzeros) runs 10 to 18 % faster, X of 64 and
        // 128 MiB up to 10 % slower, 0.5 MiB resident (13 to 27 % of the nonzeros) 30 to 60 % slower.
        const uint64_t row_bytes = (uint64_t)K * eb;
        const uint64_t budget = resident_bytes ? resident_bytes : kDefaultResidentBytes;
        const long long fit = (long long)(budget / row_bytes);
        if (pl->mark_shift > 0 && pl->num_slabs == 1 && hot_rows == 0 && !(flags & MPS_PLAN_NO_RESIDENT) && fit >= 1 &&
            fit < n && (((uint64_t)n * row_bytes >= kResidentMinXBytes && !pl->column_tiles) || resident_bytes) && pl->shape.row_shift >= 0 &&
            col_bits + 1 + bits_for(max_cold_ipt) <= 32) {
            MPS_BUILD_TRY(column_histogram());
            std::vector<int> d(h_deg);
            std::nth_element(d.begin(), d.begin() + (long)fit, d.end(), [](int a, int b) { return a > b; });
            const int thr = d[(size_t)fit];  // the (fit + 1)-th largest count: columns above it are resident
            long long above = 0, above_nnz = 0, thr_cols = 0;
            for (int c = 0; c < n; ++c) {
                const int x = h_deg[(size_t)c];
                above += x > thr;
                above_nnz += x > thr ? x : 0;
                thr_cols += x == thr;
            }
            long long ties = thr > 0 ? std::min(fit - above, thr_cols) : 0;  // columns with exactly thr nonzeros that still fit
            if (resident_bytes || (double)(above_nnz + ties * thr) >= kResidentMinShare * (double)nnz) {
                for (int c = 0; c < n; ++c) {
                    int &x = h_deg[(size_t)c];
                    const bool in = x > thr || (x == thr && ties > 0 && ties-- > 0);  // ties in column order
                    if (in) {
                        ++pl->resident_cols;
                        pl->resident_nnz += x;
                    }
                    x = in ? 0 : 1;  // from here on: the streamed flag of the column
                }
                MPS_BUILD_HIP(hipMemcpyAsync(t.deg, h_deg.data(), (size_t)n * sizeof(int), hipMemcpyHostToDevice, st));
                MPS_BUILD_HIP(hipStreamSynchronize(st));
                pl->streamed_flag = true;
            }
        }
    }

    // 5. slices
    const int W = pl->shape.num_waves;
    MPS_BUILD_TRY(dev_alloc(pl, &pl->wave_off, (size_t)W + 1));
    hipLaunchKernelGGL(slice_count_kernel, dim3((unsigned)((W + 1 + 255) / 256)), dim3(256), 0, st, pl->coord_y, pl->P, G, W,
                       pl->wave_off);
    MPS_BUILD_HIP(hipGetLastError());
    MPS_BUILD_TRY(scan_exclusive_inplace(pl->wave_off, W + 1, t.sums, st));
    int total_rounds = 0;
    MPS_BUILD_HIP(hipMemcpyAsync(&total_rounds, pl->wave_off + W, sizeof(int), hipMemcpyDeviceToHost, st));
    MPS_BUILD_HIP(hipStreamSynchronize(st));
    pl->total_rounds = total_rounds;
    const size_t slots = (size_t)total_rounds * (size_t)(G * kWindow);
    MPS_BUILD_TRY(dev_alloc(pl, &pl->slice_cols, slots));
    MPS_BUILD_TRY(dev_alloc(pl, &pl->slice_src, slots));
    if (pl->weights) {
        // no value array: the kernels add up rows of xs = col_scale * X and scale finished rows
        if (pl->mark_shift <= 0 || (hot_rows > 0 && pl->hot_mark_shift <= 0)) {
            t.drop();
            return MPS_ERR_UNSUPPORTED;
        }
        MPS_BUILD_TRY(dev_alloc(pl, &pl->col_scale, (size_t)n));
        // two spare entries: the merge path ends at row coordinate n + 1, and the kernel asks for the
        // factor of the row that would start there
        MPS_BUILD_TRY(dev_alloc(pl, &pl->row_scale, (size_t)n + 2));
        MPS_BUILD_HIP(hipMemsetAsync(pl->row_scale, 0, ((size_t)n + 2) * sizeof(float), st));
        MPS_BUILD_TRY(dev_alloc(pl, &pl->xs, (size_t)n * K));
        if (n > 0) {
            hipLaunchKernelGGL(degree_scales_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, d_row_ptr, n,
                               pl->weights - 1, pl->row_scale, pl->col_scale);
            MPS_BUILD_HIP(hipGetLastError());
        }
    } else {
        unsigned char *sv = nullptr;
        MPS_BUILD_TRY(dev_alloc(pl, &sv, (slots ? slots : 1) * (size_t)eb));
        pl->slice_vals = sv;
    }
    if (slots) {
        MPS_BUILD_HIP(hipMemsetAsync(pl->slice_cols, 0, slots * sizeof(int), st));
        MPS_BUILD_HIP(hipMemsetAsync(pl->slice_src, 0xff, slots * sizeof(int), st));
    }
    if (nnz > 0) {
        hipLaunchKernelGGL(slice_scatter_kernel, dim3((unsigned)(((long long)nnz + 255) / 256)), dim3(256), 0, st, cols_v,
                           pl->num_slabs == 1 ? nullptr : t.perm, pl->num_slabs == 1 ? nullptr : t.vrow, pl->vrow_ptr,
                           pl->n_vrows, pl->coord_x, pl->coord_y, G, pl->wave_off, nnz, max_cold_ipt,
                           hot_rows > 0 ? t.seg : nullptr, pl->num_segs, n, pl->hot_waves * G, pl->hot_mark_shift,
                           pl->mark_shift, pl->streamed_flag ? t.deg : nullptr, pl->slice_cols, pl->slice_src);
        MPS_BUILD_HIP(hipGetLastError());
    }
    if (!pl->weights) MPS_BUILD_TRY(plan_set_values(pl, d_val, st));
    if (!pl->keep_sources) {
        // only mps_plan_set_values reads the source indices again
        MPS_BUILD_HIP(hipStreamSynchronize(st));
        (void)hipFree(pl->slice_src);
        pl->slice_src = nullptr;
        pl->device_bytes -= (slots ? slots : 1) * sizeof(int);
    }

    // 6. workspace
    pl->part_bytes = part_bytes_for(n, pl->num_segs, K);
    pl->workspace_bytes = pl->part_bytes + carry_bytes_for(W, K);
    {
        unsigned char *ws = nullptr;
        MPS_BUILD_TRY(dev_alloc(pl, &ws, pl->workspace_bytes));
        pl->workspace = ws;
    }
    MPS_BUILD_HIP(hipStreamSynchronize(st));
    t.drop();
    return MPS_OK;
#undef MPS_BUILD_TRY
#undef MPS_BUILD_HIP
}

template <typename T>
int plan_spmm(const mps_plan *pl, const T *X, T *Y, unsigned phases, hipStream_t st)
{
    if (!pl || pl->elem_bytes != (int)sizeof(T)) return MPS_ERR_INVALID_ARG;
    if (pl->n_rows == 0) return MPS_OK;
    if (!X || !Y) return MPS_ERR_INVALID_ARG;
    if (!aligned_to(X, 16) || !aligned_to(Y, 16)) return MPS_ERR_ALIGNMENT;
    if (pl->rb) {
        if constexpr (sizeof(T) == 4) return mps_rb::spmm(pl->rb, X, Y, phases, st);
        else return MPS_ERR_INVALID_ARG;
    }
    if (pl->sw) return mps_sw::spmm(pl->sw, X, Y, phases, st);
    const T *vals = static_cast<const T *>(pl->slice_vals);
    void *carry = static_cast<char *>(pl->workspace) + pl->part_bytes;
    PlanLaunch how;
    how.wave_off = pl->wave_off;
    how.hot_waves = pl->hot_waves;
    how.hot_rows = pl->hot_rows;
    how.hot_cols = pl->hot_cols;
    how.seg_part_off = pl->seg_table;
    how.num_hot_segs = pl->hot_rows > 0 ? pl->num_slabs : 0;
    how.hot_lds_bytes = pl->hot_lds_bytes;
    how.hot_block_wave = pl->hot_block_wave;
    how.hot_blocks = pl->hot_blocks;
    how.mark_shift = pl->mark_shift;
    how.hot_mark_shift = pl->hot_mark_shift;
    how.streamed_flag = pl->streamed_flag;
    if (pl->weights) {
        if constexpr (sizeof(T) == 4) {
            if (phases & MPS_PHASE_PREPARE) {
                const size_t elems = (size_t)pl->n_rows * pl->K;
                if (pl->K % 4 == 0)
                    hipLaunchKernelGGL((scale_rows_kernel<4>), dim3((unsigned)((elems / 4 + 255) / 256)), dim3(256), 0, st, X,
                                       pl->col_scale, pl->xs, pl->n_rows, pl->K);
                else
                    hipLaunchKernelGGL((scale_rows_kernel<1>), dim3((unsigned)((elems + 255) / 256)), dim3(256), 0, st, X,
                                       pl->col_scale, pl->xs, pl->n_rows, pl->K);
                MPS_HIP_TRY(hipGetLastError());
            }
            X = pl->xs;
            how.pattern = true;
            how.row_scale = pl->num_segs == 1 ? pl->row_scale : nullptr;  // tiled plans: the reduce kernel scales
        } else {
            return MPS_ERR_UNSUPPORTED;
        }
    }
    if (pl->num_segs == 1)
        return launch_spmm_any<T, T>(pl->vrow_ptr, pl->slice_cols, vals, X, Y, pl->nnz, pl->K, pl->P, pl->coord_x,
                                     pl->coord_y, how, pl->shape, carry, phases, st);
    float *part = static_cast<float *>(pl->workspace);
    int rc = launch_spmm_any<T, float>(pl->vrow_ptr, pl->slice_cols, vals, X, part, pl->nnz, pl->K, pl->P, pl->coord_x,
                                       pl->coord_y, how, pl->shape, carry, phases, st);
    if (rc != MPS_OK) return rc;
    if (phases & MPS_PHASE_REDUCE) {
        const size_t per_slab = (size_t)pl->n_rows * pl->K;
        if (pl->K % 4 == 0)
            hipLaunchKernelGGL((tile_reduce_kernel<T, 4>), dim3((unsigned)((per_slab / 4 + 255) / 256)), dim3(256), 0, st,
                               part, Y, pl->n_rows, pl->K, pl->num_segs, pl->row_scale);
        else
            hipLaunchKernelGGL((tile_reduce_kernel<T, 1>), dim3((unsigned)((per_slab + 255) / 256)), dim3(256), 0, st, part,
                               Y, pl->n_rows, pl->K, pl->num_segs, pl->row_scale);
        MPS_HIP_TRY(hipGetLastError());
    }
    return MPS_OK;
}

// Row-block plan or not.  Forced: yes.  Otherwise for what the kernel is built for (fp32, K = 16)
// while X is smaller than what the slab plans treat with resident columns (R-MAT scale 22, X of
// 268 MB: 1.11 against 0.95 ms), with three kinds of matrices left to the slab plans, which the
// builder recognises once it has the matrix on the host (it then says kNotWorthwhile).  Measured on
// MI355X, ms per product, row-block with the builder's choice of steps against slab plan:
//   power law 232,965 rows x 16 per row .041/.058, x 64 .083/.146, x 492 .44/.58;
//   100,000 x 16 .027/.029; 60,000 x 16 .017/.020; 500,000 x 16 .089/.112, x 64 .226/.303;
//   1,000,000 x 16 .199/.222, x 32 .330/.410, x 60 .577/.629; 2,000,000 x 100 2.0-2.3/2.08;
//   uniform 232,965 x 32 .069/.120; 500,000 x 64 .280/.336; 1,000,000 x 60 .648/.834;
//   R-MAT scale 16 to 21, 16 per row: .018/.029, .046/.059, .184/.200, .424/.492; scale 18 x 55 .105/.157.
// (1) Many short rows (fewer than 12 per row on average, more than 2^18 rows) without busy columns
//     (kMinTableShareShortRows): uniform x 8 per row: 4,096 rows .012/.014, 20,000 .013/.015,
//     60,000 .016/.018, 200,000 .034/.034, but 1,000,000 .178/.174, 2,000,000 .363/.343,
//     4,000,000 x 4 .406/.376; with busy columns, R-MAT scale 19 x 8: .056/.071.
// (2) Columns near the diagonal (kMaxLocalShare; block-diagonal 416,349 x 5: .029/.026; banded
//     233,000 x 64 within 2,000 columns: .160/.114; 500,000 x 64 within 3,000: .427/.287): the blocks
//     idle through the steps whose column range they do not touch, and a slab plan finds such an X
//     in L2 anyway.  Where up to 8 tables of a block's own consecutive columns cover most of its
//     nonzeros, the builder makes those instead (local tables: .051/.119 and .122/.291 for the two
//     bands); only wider bands are turned away.  Bands of 30,000 and 60,000 of 233,000 columns
//     either side have a local share of 0.51 and 0.22 (.184/.120, .168/.126), 100,000 columns 0.06
//     (.133/.123: not recognised); matrices without locality 0.00.
//     The uniform rows of 8 under (1) with 4,096 to 60,000 rows are now .009/.014, .010/.015 and
//     .014/.018: a plan of one step and one round of blocks needs one launch.
// (3) A row far longer than a CU's share of the nonzeros (kMaxLongestRow; power law 262,144 x 4 with
//     a row of 50,000: .053/.034): rows are not cut across blocks.  R-MAT scale 18 x 16, whose
//     longest row is that share, is fine (.046/.059).
constexpr double kMaxLocalShare = 0.15;
constexpr double kMaxLongestRow = 2.0;
constexpr double kMinTableShareShortRows = 0.05;
bool rowblock_wanted(int n_rows, int nnz, int K, int elem_bytes, int cost, int tpw, unsigned flags)
{
    if (flags & MPS_PLAN_FORCE_ROWBLOCK) return true;
    if (flags & (MPS_PLAN_NO_ROWBLOCK | MPS_PLAN_FORCE_TILING | MPS_PLAN_NO_TILING | MPS_PLAN_FORCE_HOT | MPS_PLAN_NO_HOT)) return false;
    if (elem_bytes != 4 || K != 16 || n_rows < 1 || nnz < 1) return false;
    if ((uint64_t)n_rows * 64 >= kResidentMinXBytes) return false;
    // a caller that names a cost or partitions per wavefront of its own is tuning a slab plan: row-block plans have neither
    int default_cost = 0, max_tpw = 0;
    if (mps_default_cost(n_rows, nnz, K, elem_bytes, &default_cost) != MPS_OK || cost != default_cost) return false;
    if (mps_max_threads_per_wave(K, elem_bytes, &max_tpw) != MPS_OK || (tpw != 0 && tpw != max_tpw)) return false;
    return true;
}

// Nonzeros within `width` columns of the diagonal: 16 lanes per row, one count per workgroup added to *count.
__global__ __launch_bounds__(256) void near_diagonal_kernel(const int *__restrict__ row_ptr, const int *__restrict__ col_idx,
                                                             int n_rows, int width, unsigned long long *__restrict__ count)
{
    __shared__ unsigned block_count;
    if (threadIdx.x == 0) block_count = 0;
    __syncthreads();
    const int row = blockIdx.x * 16 + (int)(threadIdx.x >> 4), lane = (int)(threadIdx.x & 15);
    unsigned mine = 0;
    if (row < n_rows)
        for (int e = row_ptr[row] + lane; e < row_ptr[row + 1]; e += 16) {
            const int d = col_idx[e] - row;
            mine += (d <= width && d >= -width) ? 1u : 0u;
        }
    if (mine) atomicAdd(&block_count, mine);
    __syncthreads();
    if (threadIdx.x == 0 && block_count) atomicAdd(count, (unsigned long long)block_count);
}

// Sweep plan or not.  Forced: yes.  Otherwise for rows of X of 64 bytes or a multiple of 128 (and the widths that
// the comment inside sweep_wanted() adds to these), when the caller is
// not tuning a slab plan (a cost, partitions per wavefront or tiling / hot-column switches of its own) and the matrix
// is not local.  Measured on MI355X, ms per product, sweep plan against the library's other choice:
//   fp32, K = 16 (against row-block plans, slab plans where those are not built):
//     R-MAT x 16 per row, scale 16 / 18 / 20 / 21: .035/.014, .046/.044, .118-.128/.183-.197, .278/.433; scale 19 x 8 .047/.055;
//     power law 232,965 rows x 16 / 64 / 492 per row: .038/.039, .099/.085, .56/.43; 1,000,000 x 16 / 60: .146/.201, .399/.519;
//     uniform 232,965 x 32: .057/.069; 1,000,000 x 8 / 60: .133/.172, .405/.659;
//     block-diagonal 416,349 x 5: .040/.025 (row-block plan with local tables).
//   Wider rows and fp16 (against slab plans): R-MAT scale 20 x 16 at K = 32 / 64 / 128 / 256: .163-.187/.231-.272, .349/.49-.55,
//     .706/.97, 1.43/2.07; scale 18 at K = 64: .092/.119; scale 22 fp16 K = 64: .94-.97/1.11-1.15; scale 20 fp16 K = 32:
//     .178/.182; power law 232,965 x 492 at K = 32: .83/.91; x 64 at K = 64: .265/.340; uniform 1,000,000 x 8 at K = 64:
//     .365/.346; block-diagonal 416,349 x 5 at K = 64: .107/.076.
// So: with 64-byte fp32 rows, where X is 24 MiB or more (393,216 rows) - below that a row-block plan's tables serve more
// of the gathers than the sweep's locality saves; with other widths always; and never for a matrix whose nonzeros stay
// near the diagonal (kSweepMaxNearDiagonal of them within kNearDiagonalWidth columns: block-diagonal and banded
// matrices, whose X a slab plan finds in L2 anyway and which a row-block plan serves from local tables).
constexpr uint64_t kSweepMinXBytesK16 = 24ull << 20;
constexpr int kNearDiagonalWidth = 6000;
constexpr double kSweepMaxNearDiagonal = 0.6;
int sweep_wanted(const int *d_row_ptr, const int *d_col_idx, int n_rows, int nnz, int K, int elem_bytes, int cost, int tpw,
                 unsigned flags, hipStream_t st, bool *wanted, bool *near_diagonal)
{
    *wanted = false;
    *near_diagonal = false;  // set where it was looked for and found
    if (flags & MPS_PLAN_FORCE_SWEEP) {
        *wanted = true;
        return MPS_OK;
    }
    if (flags & (MPS_PLAN_NO_SWEEP | MPS_PLAN_FORCE_ROWBLOCK | MPS_PLAN_LOCAL_TABLES | MPS_PLAN_FORCE_TILING | MPS_PLAN_NO_TILING |
                 MPS_PLAN_FORCE_HOT | MPS_PLAN_NO_HOT | MPS_PLAN_NO_ROW_MARKS))
        return MPS_OK;
    // Rows of X that a sweep plan is chosen for: whole 128-byte tiles or one 64-byte tile, and, of the rows that leave
    // lanes of their last tile idle, those that fit one tile or are whole 64 bytes, as long as every lane's 16 bytes are
    // aligned.  Measured on MI355X, sweep plan against slab plan, ms per product: R-MAT scale 20 fp32 K = 8, 12, 20, 24,
    // 48: 0.122 / 0.164, 0.151 / 0.219, 0.205 / 0.240, 0.206 / 0.244, 0.347 / 0.394; the 232,965-row power-law matrix
    // K = 8, 12, 24, 48: 0.506 / 0.683, 0.563 / 0.924, 0.842 / 1.035, 1.56 / 1.72; R-MAT scale 22 fp16 K = 24, 40:
    // 0.826 / 0.860, 1.03 / 1.17.  Left to the slab plans: rows of several tiles that start anywhere in a 128-byte
    // line (fp32 K = 100: 0.925 / 0.894 and 3.59 / 3.51) and rows whose pitch is no multiple of 16 bytes, where a
    // lane's 16 bytes lie across two aligned ones (fp32 K = 41: 0.494 / 0.526; fp16 K = 100: 2.81 / 2.31).
    const long long row_bytes = (long long)K * elem_bytes;
    const bool whole_tiles = row_bytes == 64 || row_bytes % 128 == 0;
    const bool idle_lanes_pay = row_bytes % 16 == 0 && (row_bytes < 128 || row_bytes % 64 == 0);
    if (n_rows < 1 || nnz < 1 || !(whole_tiles || idle_lanes_pay)) return MPS_OK;
    if (n_rows > (1 << 26)) return MPS_OK;  // an entry word keeps 6 bits for the accumulator row
    int default_cost = 0, max_tpw = 0;
    if (mps_default_cost(n_rows, nnz, K, elem_bytes, &default_cost) != MPS_OK || cost != default_cost) return MPS_OK;
    if (mps_max_threads_per_wave(K, elem_bytes, &max_tpw) != MPS_OK || (tpw != 0 && tpw != max_tpw)) return MPS_OK;
    if (row_bytes == 64 && elem_bytes == 4 && (uint64_t)n_rows * 64 < kSweepMinXBytesK16) return MPS_OK;
    // the kernel below follows row_ptr into col_idx: only on arrays that have been checked
    const int vrc = mps_csr_validate(d_row_ptr, d_col_idx, n_rows, n_rows, nnz, st);
    if (vrc != MPS_OK) return vrc;
    unsigned long long *d_count = nullptr, near = 0;
    MPS_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&d_count), sizeof(unsigned long long)));
    hipError_t e = hipMemsetAsync(d_count, 0, sizeof(unsigned long long), st);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(near_diagonal_kernel, dim3((unsigned)((n_rows + 15) / 16)), dim3(256), 0, st, d_row_ptr, d_col_idx,
                           n_rows, kNearDiagonalWidth, d_count);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(&near, d_count, sizeof(near), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    (void)hipFree(d_count);
    if (e != hipSuccess) return MPS_ERR_HIP + (int)e;
    // (a matrix narrower than the window is all "near the diagonal": what counts then is whether X fits an L2,
    // and that case never gets here with 64-byte rows; wider rows of a small matrix keep the sweep)
    const bool small = n_rows <= 2 * kNearDiagonalWidth;
    *wanted = small || (double)near < kSweepMaxNearDiagonal * (double)nnz;
    *near_diagonal = !*wanted;
    return MPS_OK;
}

}  // namespace

extern "C" {

int mps_tile_shape(int n_rows, int nnz, int K, int elem_bytes, size_t slab_bytes, int *num_slabs_out,
                   int *slab_cols_out)
{
    if (!num_slabs_out || !slab_cols_out || n_rows < 0 || nnz < 0 || K < 1) return MPS_ERR_INVALID_ARG;
    if (elem_bytes != 4 && elem_bytes != 2) return MPS_ERR_INVALID_ARG;
    pick_tile_shape(n_rows, nnz, K, elem_bytes, slab_bytes, -1.0, num_slabs_out, slab_cols_out);
    return MPS_OK;
}

int mps_plan_create(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n_rows, int nnz, int K,
                    int elem_bytes, int cost, int tpw, unsigned flags, size_t slab_bytes, void *stream,
                    mps_plan **plan_out)
{
    mps_plan_options opt{};
    opt.flags = flags;
    opt.slab_bytes = slab_bytes;
    return mps_plan_create_ex(d_row_ptr, d_col_idx, d_val, n_rows, nnz, K, elem_bytes, cost, tpw, &opt, stream, plan_out);
}

int mps_plan_create_ex(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n_rows, int nnz, int K,
                       int elem_bytes, int cost, int tpw, const mps_plan_options *options, void *stream,
                       mps_plan **plan_out)
{
    if (!plan_out) return MPS_ERR_INVALID_ARG;
    *plan_out = nullptr;
    if (!d_row_ptr || n_rows < 0 || nnz < 0 || K < 1 || cost <= 0 || tpw < 0) return MPS_ERR_INVALID_ARG;
    if (elem_bytes != 4 && elem_bytes != 2) return MPS_ERR_INVALID_ARG;
    mps_plan_options opt{};
    if (options) opt = *options;
    if (opt.degree_weights < 0 || opt.degree_weights > 2) return MPS_ERR_INVALID_ARG;
    if (nnz > 0 && (!d_col_idx || (!d_val && !opt.degree_weights))) return MPS_ERR_INVALID_ARG;
    if ((long long)n_rows + 1 + nnz > INT_MAX) return MPS_ERR_UNSUPPORTED;
    if (opt.degree_weights) {
        // built for fp32 and the slab kernels; the source indices serve new values only
        if (elem_bytes != 4 || (opt.flags & (MPS_PLAN_FORCE_ROWBLOCK | MPS_PLAN_FORCE_SWEEP))) return MPS_ERR_UNSUPPORTED;
        opt.flags |= MPS_PLAN_NO_ROWBLOCK | MPS_PLAN_NO_SWEEP | MPS_PLAN_NO_SOURCES;
        opt.flags &= ~MPS_PLAN_NO_ROW_MARKS;
    }
    const unsigned flags = opt.flags;
    const size_t slab_bytes = opt.slab_bytes;
    if ((flags & MPS_PLAN_FORCE_ROWBLOCK) && (flags & (MPS_PLAN_NO_ROWBLOCK | MPS_PLAN_FORCE_TILING))) return MPS_ERR_INVALID_ARG;
    if ((flags & MPS_PLAN_FORCE_SWEEP) && (flags & (MPS_PLAN_NO_SWEEP | MPS_PLAN_FORCE_TILING | MPS_PLAN_FORCE_ROWBLOCK))) return MPS_ERR_INVALID_ARG;
    mps_plan *pl = new (std::nothrow) mps_plan;
    if (!pl) return MPS_ERR_UNSUPPORTED;
    pl->n_rows = n_rows;
    pl->nnz = nnz;
    pl->K = K;
    pl->elem_bytes = elem_bytes;
    pl->cost = cost;
    pl->keep_sources = !(flags & MPS_PLAN_NO_SOURCES);
    pl->weights = opt.degree_weights;
    bool want_sweep = false, near_diagonal = false;
    if (!opt.degree_weights) {
        const int src = sweep_wanted(d_row_ptr, d_col_idx, n_rows, nnz, K, elem_bytes, cost, tpw, flags,
                                     static_cast<hipStream_t>(stream), &want_sweep, &near_diagonal);
        if (src != MPS_OK) {
            plan_free(pl);
            return src;
        }
    }
    if (want_sweep) {
        if (n_rows < 1 || ((long long)K * elem_bytes) % 4 != 0) {
            plan_free(pl);
            return MPS_ERR_UNSUPPORTED;
        }
        // the builder indexes X and its own tables by column id
        if (flags & MPS_PLAN_FORCE_SWEEP) {
            int vrc = mps_csr_validate(d_row_ptr, d_col_idx, n_rows, n_rows, nnz, stream);
            if (vrc != MPS_OK) {
                plan_free(pl);
                return vrc;
            }
        }
        mps_sw::BuildParams bp;
        bp.piece = opt.sweep_piece;
        bp.acc_rows = opt.sweep_acc_rows;
        bp.num_cus = opt.sweep_panels_per_round;  // 0: ask the device
        bp.together = opt.sweep_together;
        bp.elem_bytes = elem_bytes;
        bp.keep_src = pl->keep_sources;
        bp.host_build = (flags & MPS_PLAN_HOST_BUILD) != 0;
        int rc = mps_sw::create(d_row_ptr, d_col_idx, d_val, n_rows, nnz, K, bp, static_cast<hipStream_t>(stream), &pl->sw);
        if (rc == MPS_OK) {
            pl->device_bytes = mps_sw::device_bytes_of(pl->sw);
            make_spmm_shape(n_rows, K, 1, 0, elem_bytes, pl->shape);
            *plan_out = pl;
            return MPS_OK;
        }
        if (rc != MPS_ERR_UNSUPPORTED || (flags & MPS_PLAN_FORCE_SWEEP)) {
            plan_free(pl);
            return rc;
        }
        // (column ids that leave no room for the accumulator row in an entry word: another kind of plan below)
    }
    if (rowblock_wanted(n_rows, nnz, K, elem_bytes, cost, tpw, flags)) {
        if (elem_bytes != 4 || K != 16 || n_rows < 1) {
            plan_free(pl);
            return MPS_ERR_UNSUPPORTED;
        }
        // the builder's tables are indexed by column id
        int vrc = mps_csr_validate(d_row_ptr, d_col_idx, n_rows, n_rows, nnz, stream);
        if (vrc != MPS_OK) {
            plan_free(pl);
            return vrc;
        }
        mps_rb::BuildParams bp;
        bp.steps = opt.rowblock_steps;
        bp.table_rows = opt.rowblock_table_rows;
        bp.block_rows = opt.rowblock_block_rows;
        bp.num_cus = opt.rowblock_blocks_per_round;  // 0: ask the device
        bp.keep_src = pl->keep_sources;
        bp.local_tables = (flags & MPS_PLAN_LOCAL_TABLES) != 0;
        // (a matrix that keeps to its diagonal gets local tables, which the host passes lay out: straight there)
        bp.host_build = (flags & MPS_PLAN_HOST_BUILD) != 0 || near_diagonal;
        if (!(flags & MPS_PLAN_FORCE_ROWBLOCK)) {
            bp.max_local_share = kMaxLocalShare;
            bp.max_longest_row = kMaxLongestRow;
            bp.min_table_share_short_rows = kMinTableShareShortRows;
        }
        int rc = mps_rb::create(d_row_ptr, d_col_idx, static_cast<const float *>(d_val), n_rows, nnz, K, bp,
                                static_cast<hipStream_t>(stream), &pl->rb);
        if (rc == MPS_OK) {
            pl->device_bytes = mps_rb::device_bytes_of(pl->rb);
            make_spmm_shape(n_rows, K, 1, 0, elem_bytes, pl->shape);
            *plan_out = pl;
            return MPS_OK;
        }
        if (rc != mps_rb::kNotWorthwhile) {
            plan_free(pl);
            return rc;
        }
        // short rows, one very long row, or local columns that no table of a block's own covers: the slab plan below
    }
    int rc;
    try {
        rc = plan_build(pl, d_row_ptr, d_col_idx, d_val, flags, slab_bytes, opt.resident_bytes, tpw,
                        static_cast<hipStream_t>(stream));
    } catch (const std::bad_alloc &) {  // host-side tables of the build
        rc = MPS_ERR_UNSUPPORTED;
    }
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
    info->num_segments = plan->num_segs;
    info->hot_rows = plan->hot_rows;
    info->hot_waves = plan->hot_waves;
    info->hot_nnz = plan->hot_nnz;
    info->hot_cost = plan->hot_cost;
    info->mark_shift = plan->mark_shift;
    info->hot_mark_shift = plan->hot_mark_shift;
    info->resident_cols = plan->resident_cols;
    info->resident_nnz = plan->resident_nnz;
    info->hot_blocks = plan->hot_blocks;
    info->rowblock_steps = info->rowblock_table_rows = info->rowblock_blocks = info->rowblock_acc_rows = 0;
    info->rowblock_hot_slots = info->rowblock_cold_slots = 0;
    info->rowblock_cold_index_bits = 0;
    info->rowblock_local_tables = 0;
    info->sweep_panels = info->sweep_acc_rows = info->sweep_lanes = info->sweep_tiles = info->sweep_col_bits = 0;
    info->sweep_piece = info->sweep_together = info->sweep_split_rows = info->sweep_partial_rows = info->sweep_listed_rows = 0;
    info->sweep_rounds = info->sweep_slots = 0;
    info->built_on_device = 1;
    if (plan->sw) {
        info->num_slabs = 1;
        info->slab_cols = plan->n_rows;
        mps_sw::fill_info(mps_sw::layout_of(plan->sw), info);
        info->built_on_device = mps_sw::built_on_device(plan->sw) ? 1 : 0;
    }
    if (plan->rb) {
        const mps_rb::Layout &L = mps_rb::layout_of(plan->rb);
        info->num_slabs = 1;
        info->slab_cols = plan->n_rows;
        info->hot_nnz = L.hot_nnz;
        info->mark_shift = L.cold_bits;
        info->hot_mark_shift = L.hot_bits;
        info->rowblock_steps = L.steps;
        info->rowblock_table_rows = L.table_rows;
        info->rowblock_blocks = L.num_blocks;
        info->rowblock_acc_rows = L.acc_rows;
        info->rowblock_hot_slots = L.hot_rounds * mps_rb::kRoundEntries;
        info->rowblock_cold_slots = L.cold_rounds * mps_rb::kRoundEntries;
        info->rowblock_cold_index_bits = L.cold_index_bits;
        info->rowblock_local_tables = L.table_base.empty() ? 0 : 1;
        info->built_on_device = mps_rb::built_on_device(plan->rb) ? 1 : 0;
    }
    return MPS_OK;
}

int mps_plan_set_values(mps_plan *plan, const void *d_val, void *stream)
{
    if (!plan || (plan->nnz > 0 && !d_val)) return MPS_ERR_INVALID_ARG;
    if (!plan->keep_sources || plan->weights) return MPS_ERR_UNSUPPORTED;
    if (plan->rb) return mps_rb::set_values(plan->rb, static_cast<const float *>(d_val), static_cast<hipStream_t>(stream));
    if (plan->sw) return mps_sw::set_values(plan->sw, d_val, static_cast<hipStream_t>(stream));
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
    case MPS_PLAN_ARRAY_SLICE_SRC: src = plan->slice_src; have = plan->slice_src ? slots * sizeof(int) : 0; break;
    case MPS_PLAN_ARRAY_SLICE_VALS: src = plan->slice_vals; have = plan->slice_vals ? slots * (size_t)plan->elem_bytes : 0; break;
    case MPS_PLAN_ARRAY_HOT_COLS:
        src = plan->hot_cols;
        have = (size_t)(plan->hot_rows > 0 ? plan->num_slabs : 0) * (size_t)plan->hot_rows * sizeof(int);
        break;
    default:
        if (which >= MPS_PLAN_ARRAY_SW_PANEL_PTR && which <= MPS_PLAN_ARRAY_SW_SPLIT_PTR) {
            if (!plan->sw) return MPS_ERR_INVALID_ARG;
            src = mps_sw::device_array(plan->sw, which, &have);
            break;
        }
        if (!plan->rb) return MPS_ERR_INVALID_ARG;
        src = mps_rb::device_array(plan->rb, which, &have);
        if (!src && have == 0 && (which < MPS_PLAN_ARRAY_RB_BLOCK_ROW || which > MPS_PLAN_ARRAY_RB_TABLE_BASE)) return MPS_ERR_INVALID_ARG;
        break;
    }
    if ((plan->rb || plan->sw) && which < MPS_PLAN_ARRAY_RB_BLOCK_ROW) return MPS_ERR_INVALID_ARG;
    if (bytes != have) return MPS_ERR_INVALID_ARG;
    if (have == 0) return MPS_OK;
    MPS_HIP_TRY(hipMemcpy(host_dst, src, have, hipMemcpyDeviceToHost));
    return MPS_OK;
}

int mps_plan_spmm_f32(const mps_plan *plan, const float *d_X, float *d_Y, void *stream)
{
    return plan_spmm<float>(plan, d_X, d_Y, MPS_PHASE_PREPARE | MPS_PHASE_MAIN | MPS_PHASE_FIXUP | MPS_PHASE_REDUCE,
                            static_cast<hipStream_t>(stream));
}

int mps_plan_spmm_f16(const mps_plan *plan, const uint16_t *d_X, uint16_t *d_Y, void *stream)
{
    return plan_spmm<half_t>(plan, reinterpret_cast<const half_t *>(d_X), reinterpret_cast<half_t *>(d_Y),
                             MPS_PHASE_PREPARE | MPS_PHASE_MAIN | MPS_PHASE_FIXUP | MPS_PHASE_REDUCE, static_cast<hipStream_t>(stream));
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

int mps_plan_autotune(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n_rows, int nnz, int K,
                      int elem_bytes, const void *d_X, void *d_Y, int repeats, void *stream, mps_tune_result *best_out,
                      mps_tune_result *tried_out, int *n_tried_io)
{
    if (!best_out || !d_row_ptr || n_rows < 0 || nnz < 0 || K < 1) return MPS_ERR_INVALID_ARG;
    if (tried_out && !n_tried_io) return MPS_ERR_INVALID_ARG;
    if (n_rows > 0 && (!d_X || !d_Y)) return MPS_ERR_INVALID_ARG;
    if (repeats < 1) repeats = 5;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int max_tpw = 0, dflt = 0;
    int rc = mps_max_threads_per_wave(K, elem_bytes, &max_tpw);
    if (rc != MPS_OK) return rc;
    if ((rc = mps_default_cost(n_rows, nnz, K, elem_bytes, &dflt)) != MPS_OK) return rc;
    // what the reference's authors swept by hand: cost and partitions per wave
    // (src/MergePathSpMM.cu:121-122), plus this library's own switch
    // (slab plans: a row-block plan has neither a cost nor partitions per wavefront, it is one candidate of its own)
    mps_tune_result cand[20];
    int n_cand = 0;
    const unsigned slab = MPS_PLAN_NO_ROWBLOCK | MPS_PLAN_NO_SWEEP;
    const int costs[] = {16, 24, 32, 48, 64, 96, 128, 256};
    for (int c : costs) cand[n_cand++] = {c, max_tpw, slab, 0.f, 0};
    if (max_tpw >= 2) cand[n_cand++] = {dflt, max_tpw / 2, slab, 0.f, 0};
    cand[n_cand++] = {dflt, max_tpw, slab | MPS_PLAN_NO_HOT, 0.f, 0};
    cand[n_cand++] = {dflt, max_tpw, slab | MPS_PLAN_NO_TILING, 0.f, 0};
    if (elem_bytes == 4 && K == 16 && n_rows >= 1 && nnz >= 1 && (uint64_t)n_rows * 64 < kResidentMinXBytes)
        cand[n_cand++] = {dflt, max_tpw, MPS_PLAN_FORCE_ROWBLOCK, 0.f, 0};
    if (((long long)K * elem_bytes) % 64 == 0 && n_rows >= 1 && nnz >= 1 && n_rows <= (1 << 26))
        cand[n_cand++] = {dflt, max_tpw, MPS_PLAN_FORCE_SWEEP, 0.f, 0};
    // slab sizes the model does not pick on its own: larger slabs pay on skewed graphs
    // (not those the model puts 50 % behind the untiled plan: thousands of slabs for a matrix with short rows)
    const double untiled_ps = modelled_ps(n_rows, nnz, K, elem_bytes, 1, n_rows, -1.0);
    for (unsigned long long mib : {3ull, 6ull, 12ull, 24ull}) {
        const unsigned long long row_bytes = (unsigned long long)K * elem_bytes;
        if ((unsigned long long)n_rows * row_bytes <= 2 * (mib << 20)) continue;
        unsigned long long cols = (mib << 20) / row_bytes / 64 * 64;  // what MPS_PLAN_FORCE_TILING makes of the size
        if (cols < 64) cols = 64;
        const unsigned long long slabs = ((unsigned long long)n_rows + cols - 1) / cols;
        if (modelled_ps(n_rows, nnz, K, elem_bytes, (int)slabs, (int)cols, -1.0) > 1.5 * untiled_ps) continue;
        cand[n_cand++] = {dflt, max_tpw, slab | MPS_PLAN_FORCE_TILING | MPS_PLAN_NO_HOT, 0.f, mib << 20};
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    MPS_HIP_TRY(hipEventCreate(&e0));
    hipError_t he = hipEventCreate(&e1);
    if (he != hipSuccess) {
        (void)hipEventDestroy(e0);
        return MPS_ERR_HIP + (int)he;
    }
    mps_tune_result best{0, 0, 0u, 0.f, 0};
    int tried = 0;
    const int cap = (tried_out && n_tried_io) ? *n_tried_io : 0;
    rc = MPS_OK;
    for (int ci = 0; ci < n_cand; ++ci) {
        mps_tune_result &c = cand[ci];
        mps_plan *pl = nullptr;
        rc = mps_plan_create(d_row_ptr, d_col_idx, d_val, n_rows, nnz, K, elem_bytes, c.cost, c.threads_per_wave, c.flags,
                             (size_t)c.slab_bytes, stream, &pl);
        if ((c.flags & (MPS_PLAN_FORCE_TILING | MPS_PLAN_FORCE_ROWBLOCK | MPS_PLAN_FORCE_SWEEP)) && (rc == MPS_ERR_UNSORTED || rc == MPS_ERR_UNSUPPORTED)) {
            rc = MPS_OK;  // this matrix cannot be tiled or blocked that way: not a candidate
            continue;
        }
        if (rc != MPS_OK) break;
        const unsigned all = MPS_PHASE_PREPARE | MPS_PHASE_MAIN | MPS_PHASE_FIXUP | MPS_PHASE_REDUCE;
        for (int i = 0; i < 2 && rc == MPS_OK; ++i) rc = mps_plan_spmm_phases(pl, d_X, d_Y, all, stream);
        if (rc == MPS_OK) he = hipEventRecord(e0, st);
        for (int i = 0; i < repeats && rc == MPS_OK; ++i) rc = mps_plan_spmm_phases(pl, d_X, d_Y, all, stream);
        if (rc == MPS_OK && he == hipSuccess) he = hipEventRecord(e1, st);
        if (rc == MPS_OK && he == hipSuccess) he = hipEventSynchronize(e1);
        float ms = 0.f;
        if (rc == MPS_OK && he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
        mps_plan_destroy(pl);
        if (rc == MPS_OK && he != hipSuccess) rc = MPS_ERR_HIP + (int)he;
        if (rc != MPS_OK) break;
        c.ms = ms / (float)repeats;
        if (best.cost == 0 || c.ms < best.ms) best = c;
        if (tried < cap) tried_out[tried] = c;
        ++tried;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != MPS_OK) return rc;
    if (n_tried_io) *n_tried_io = tried;
    *best_out = best;
    return MPS_OK;
}

}  // extern "C"
