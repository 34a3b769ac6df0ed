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
// Column-slab tiling.  The dense-row gathers are served by the L2 of the XCD
// the wavefront runs on (4 MiB each); a feature matrix larger than that
// misses to the fabric, whose request rate then bounds the kernel.  The tiled
// entry points reorder the nonzeros slab-major (all rows of column slab 0,
// then slab 1, ...), so that at any moment the running wavefronts gather from
// one ~2 MiB slab of X, and run the same merge-path kernel over the resulting
// num_slabs * n_rows "virtual rows"; a last kernel adds the per-slab partial
// rows in slab order.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>
#include <cstdlib>

#include "mpspmm.h"
#include "mpspmm_internal.h"

#define MPS_HIP_TRY(expr)                                       \
    do {                                                        \
        hipError_t e_ = (expr);                                 \
        if (e_ != hipSuccess) return MPS_ERR_HIP + (int)e_;     \
    } while (0)

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr int kWindow = 16;  // nonzeros staged per lane-group per round

using half_t = _Float16;
typedef half_t half8_t __attribute__((ext_vector_type(8)));
typedef half_t half4_t __attribute__((ext_vector_type(4)));
// 4-byte aligned 16-byte vectors: windows start at any nonzero index
typedef int int4u_t __attribute__((ext_vector_type(4), aligned(4)));
typedef float float4u_t __attribute__((ext_vector_type(4), aligned(4)));
typedef half_t half4u_t __attribute__((ext_vector_type(4), aligned(2)));

// LDS traffic here is private to one wavefront (each wave owns its slice), and
// a wave's LDS operations execute in order, so a compiler-level barrier is all
// that is needed between its writes and its reads.
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------
// Per-(element type, vector width) access to the dense input.
// ---------------------------------------------------------------------------
template <typename T, int VEC>
struct XOps;

template <>
struct XOps<float, 4> {
    using Raw = float4;
    static __device__ __forceinline__ void fma(float (&acc)[4], float v, const Raw &r)
    {
        acc[0] = __builtin_fmaf(v, r.x, acc[0]);
        acc[1] = __builtin_fmaf(v, r.y, acc[1]);
        acc[2] = __builtin_fmaf(v, r.z, acc[2]);
        acc[3] = __builtin_fmaf(v, r.w, acc[3]);
    }
};

template <>
struct XOps<float, 1> {
    using Raw = float;
    static __device__ __forceinline__ void fma(float (&acc)[1], float v, const Raw &r)
    {
        acc[0] = __builtin_fmaf(v, r, acc[0]);
    }
};

template <>
struct XOps<half_t, 8> {
    using Raw = half8_t;
    static __device__ __forceinline__ void fma(float (&acc)[8], float v, const Raw &r)
    {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(v, (float)r[i], acc[i]);
    }
};

template <>
struct XOps<half_t, 1> {
    using Raw = half_t;
    static __device__ __forceinline__ void fma(float (&acc)[1], float v, const Raw &r)
    {
        acc[0] = __builtin_fmaf(v, (float)r, acc[0]);
    }
};

// VEC accumulators -> VEC adjacent outputs (fp32 or fp16), one vector store
// where the width allows.
template <int VEC>
__device__ __forceinline__ void store_acc(float *p, const float (&acc)[VEC])
{
    if constexpr (VEC % 4 == 0) {
#pragma unroll
        for (int i = 0; i < VEC; i += 4)
            *reinterpret_cast<float4 *>(p + i) = make_float4(acc[i], acc[i + 1], acc[i + 2], acc[i + 3]);
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) p[i] = acc[i];
    }
}
template <int VEC>
__device__ __forceinline__ void store_acc(half_t *p, const float (&acc)[VEC])
{
    if constexpr (VEC == 8) {
        half8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (half_t)acc[i];
        *reinterpret_cast<half8_t *>(p) = o;
    } else if constexpr (VEC == 4) {
        half4_t o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = (half_t)acc[i];
        *reinterpret_cast<half4_t *>(p) = o;
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) p[i] = (half_t)acc[i];
    }
}

// Address of the VEC columns a lane owns in row `c` of X.  POW2: the row
// pitch is a power of two and the matrix is below 4 GiB, so the byte offset
// is one shift-or in 32 bits (the load then takes its base from SGPRs).
template <typename T, int VEC, bool POW2>
struct Gather {
    using Raw = typename XOps<T, VEC>::Raw;
    const char *xb;
    size_t row_bytes;
    unsigned col_byte;
    int row_shift;
    __device__ __forceinline__ Raw load(int c) const
    {
        if constexpr (POW2) {
            unsigned off = ((unsigned)c << row_shift) | col_byte;
            return *reinterpret_cast<const Raw *>(xb + off);
        } else {
            size_t off = (size_t)c * row_bytes + col_byte;
            return *reinterpret_cast<const Raw *>(xb + off);
        }
    }
};

// Four consecutive nonzeros of a window, as registers.
struct Win {
    int4 c;
    float4 v;
};

__device__ __forceinline__ float4 load_val4(const float *p)
{
    float4u_t t = __builtin_nontemporal_load(reinterpret_cast<const float4u_t *>(p));
    return make_float4(t[0], t[1], t[2], t[3]);
}
__device__ __forceinline__ float4 load_val4(const half_t *p)
{
    half4u_t h = __builtin_nontemporal_load(reinterpret_cast<const half4u_t *>(p));
    return make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
}

// Nonzeros [i0, i0 + 4) of col_idx / val (those below nnz).  The sparse
// stream is read once: non-temporal loads keep it from displacing X in L2.
template <typename T>
__device__ __forceinline__ Win load_win(const int *__restrict__ col_idx, const T *__restrict__ val, int nnz, int i0)
{
    Win w;
    w.c = make_int4(0, 0, 0, 0);
    w.v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i0 + 3 < nnz) {
        int4u_t t = __builtin_nontemporal_load(reinterpret_cast<const int4u_t *>(col_idx + i0));
        w.c = make_int4(t[0], t[1], t[2], t[3]);
        w.v = load_val4(val + i0);
    } else {
        if (i0 + 0 < nnz) { w.c.x = col_idx[i0 + 0]; w.v.x = (float)val[i0 + 0]; }
        if (i0 + 1 < nnz) { w.c.y = col_idx[i0 + 1]; w.v.y = (float)val[i0 + 1]; }
        if (i0 + 2 < nnz) { w.c.z = col_idx[i0 + 2]; w.v.z = (float)val[i0 + 2]; }
    }
    return w;
}

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

// The six arrays of generate_mp_sched (src/MergePathSpMM.cu:336-376), from the
// coordinates, zero-means-none encoding included.
__global__ __launch_bounds__(256) void mp_schedule_legacy_kernel(
    const int *__restrict__ row_ptr, int P, const int *__restrict__ coord_x,
    const int *__restrict__ coord_y, int *__restrict__ feature_start_all,
    int *__restrict__ feature_start_num, int *__restrict__ feature_end_all,
    int *__restrict__ feature_end_num, int *__restrict__ start_row_all, int *__restrict__ end_row_all)
{
    int core_id = blockIdx.x * blockDim.x + threadIdx.x;
    if (core_id >= P) return;
    int start = coord_x[core_id] - 1;
    int end = coord_x[core_id + 1] - 1;
    if (start < 0) start = 0;
    int num_features = 0;
    int feature_start = coord_y[core_id];
    if (row_ptr[start] == feature_start) feature_start = 0;
    if (core_id == 0) feature_start = 0;
    int feature_end = coord_y[core_id + 1];
    if (row_ptr[end] == feature_end) feature_end = 0;
    if (feature_start != 0) {
        if (start == end && feature_end != 0) {
            num_features = feature_end - feature_start;
            feature_end = 0;
        } else {
            num_features = row_ptr[start + 1] - feature_start;
        }
    }
    int num_features_end = 0;
    if (feature_end != 0) {
        num_features_end = feature_end - row_ptr[end];
        feature_end = row_ptr[end];
    }
    feature_start_all[core_id] = feature_start;
    feature_end_all[core_id] = feature_end;
    feature_start_num[core_id] = num_features;
    feature_end_num[core_id] = num_features_end;
    start_row_all[core_id] = start;
    end_row_all[core_id] = end;
}

// ---------------------------------------------------------------------------
// Merge-path SpMM, main kernel.
// ---------------------------------------------------------------------------
template <typename T, typename TOut, int VEC, bool POW2, int BATCH>
__global__ __launch_bounds__(kBlock) void mp_spmm_kernel(
    const int *__restrict__ row_ptr, const int *__restrict__ col_idx, const T *__restrict__ val,
    const T *__restrict__ X, TOut *__restrict__ Y, const int *__restrict__ coord_x,
    const int *__restrict__ coord_y, int nnz, int K, int P, int lanes_log2, int tpw, int num_waves,
    int row_shift, int *__restrict__ ws_head_row, float *__restrict__ ws_head, float *__restrict__ ws_tail)
{
    using XO = XOps<T, VEC>;
    using Raw = typename XO::Raw;
    constexpr int kCombine = 64 * VEC;  // floats per wave for heads (and for tails)
    constexpr int kSlice = (2 * kCombine > 2 * 16 * kWindow) ? 2 * kCombine : 2 * 16 * kWindow;
    __shared__ float s_buf[kWavesPerBlock][kSlice];
    __shared__ int s_hrow[kWavesPerBlock][16];

    const int wib = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int w = blockIdx.x * kWavesPerBlock + wib;
    if (w >= num_waves) return;

    const int L = 1 << lanes_log2;
    const int g = lane >> lanes_log2;
    const int s = lane & (L - 1);
    const int KT = L * VEC;  // columns covered by one pass of the wave
    const int kcol = blockIdx.y * KT + s * VEC;
    const bool col_ok = kcol < K;
    // lanes beyond K gather column 0 (a valid address) and never store
    const Gather<T, VEC, POW2> gx{reinterpret_cast<const char *>(X), (size_t)K * sizeof(T),
                                  col_ok ? (unsigned)(kcol * sizeof(T)) : 0u, row_shift};

    int *s_col = reinterpret_cast<int *>(&s_buf[wib][0]) + g * kWindow;
    float *s_val = &s_buf[wib][16 * kWindow] + g * kWindow;

    const int p = w * tpw + g;
    const bool part_ok = (g < tpw) && (p < P);
    int x = 1, x_end = 1, y_begin = 0, y_end = 0;
    if (part_ok) {
        x = max(coord_x[p], 1);
        x_end = coord_x[p + 1];
        y_begin = coord_y[p];
        y_end = coord_y[p + 1];
    }
    // Row x - 1 is in progress; it ends where nonzero index row_ptr[x] begins.
    // The two row ends after it are loaded ahead, so that finishing a row does
    // not wait on memory.
    auto row_end_at = [&](int xx) { return (xx < x_end) ? row_ptr[xx] : INT_MAX; };
    int row_end = row_end_at(x), row_end1 = row_end_at(x + 1), row_end2 = row_end_at(x + 2);

    float acc[VEC], head[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) { acc[i] = 0.f; head[i] = 0.f; }
    int head_row = -1;

    auto emit = [&]() {
        const int row = x - 1;
        if (head_row < 0) {
            head_row = row;
#pragma unroll
            for (int i = 0; i < VEC; ++i) head[i] = acc[i];
        } else if (col_ok) {
            store_acc<VEC>(Y + (size_t)row * K + kcol, acc);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        ++x;
        row_end = row_end1;
        row_end1 = row_end2;
        row_end2 = row_end_at(x + 2);
    };

    int wbase = y_begin;
    Win pw;
    pw.c = make_int4(0, 0, 0, 0);
    pw.v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (s < 4 && wbase < y_end) pw = load_win<T>(col_idx, val, nnz, wbase + 4 * s);

    while (__any(wbase < y_end)) {
        const int nvalid = min(kWindow, y_end - wbase);  // <= 0 for a group that is done
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
                // next window: in flight while this one is consumed
                const int nb = wbase + kWindow;
                if (s < 4 && nb < y_end) pw = load_win<T>(col_idx, val, nnz, nb + 4 * s);
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                if (b + j < nvalid) {
                    const int idx = wbase + b + j;
                    while (idx == row_end) emit();
                    XO::fma(acc, vals[j], xr[j]);
                }
            }
        }
        wbase += kWindow;
        wave_lds_sync();
    }
    while (x < x_end) emit();  // rows that end exactly where the partition ends

    // ---- combine the groups of this wavefront -------------------------------
    float *heads = &s_buf[wib][0];
    float *tails = heads + kCombine;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        heads[g * KT + s * VEC + i] = head[i];
        tails[g * KT + s * VEC + i] = acc[i];
    }
    if (s == 0) s_hrow[wib][g] = head_row;
    wave_lds_sync();

    const int ng = min(tpw, P - w * tpw);
    for (int c = lane; c < KT; c += 64) {
        const int kc = blockIdx.y * KT + c;
        const bool kc_ok = kc < K;
        float carry = 0.f;
        bool first = true;
        for (int gg = 0; gg < ng; ++gg) {
            const int hr = s_hrow[wib][gg];
            const float t = tails[gg * KT + c];
            if (hr >= 0) {
                const float v = heads[gg * KT + c] + carry;
                if (first) {
                    if (kc_ok) ws_head[(size_t)w * K + kc] = v;
                    if (kc == 0) ws_head_row[w] = hr;
                    first = false;
                } else if (kc_ok) {
                    Y[(size_t)hr * K + kc] = (TOut)v;
                }
                carry = t;
            } else {
                carry += t;
            }
        }
        if (first && kc == 0) ws_head_row[w] = -1;
        if (kc_ok) ws_tail[(size_t)w * K + kc] = carry;
    }
}

// Carry-out fix-up: the first row that ends inside wavefront w also received
// nonzeros from the wavefronts before it, back to (and including) the nearest
// one that itself saw a row end.
template <typename TOut>
__global__ __launch_bounds__(256) void mp_fixup_kernel(const int *__restrict__ ws_head_row,
                                                        const float *__restrict__ ws_head,
                                                        const float *__restrict__ ws_tail,
                                                        TOut *__restrict__ Y, int num_waves, int K)
{
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long w64 = idx / K;
    if (w64 >= num_waves) return;
    const int w = (int)w64;
    const int k = (int)(idx - w64 * K);
    const int hr = ws_head_row[w];
    if (hr < 0) return;
    float sum = ws_head[(size_t)w * K + k];
    int j = w - 1;
    while (j >= 0) {
        // four records at a time so that their loads overlap
        float t[4];
        int h[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int jj = j - u;
            t[u] = jj >= 0 ? ws_tail[(size_t)jj * K + k] : 0.f;
            h[u] = jj >= 0 ? ws_head_row[jj] : 0;
        }
        bool done = false;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (!done) {
                sum += t[u];
                if (h[u] >= 0) done = true;
            }
        }
        if (done) break;
        j -= 4;
    }
    Y[(size_t)hr * K + k] = (TOut)sum;
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
// Exclusive prefix sum of an int array, in place (three launches).
// ---------------------------------------------------------------------------
constexpr int kScanThreads = 1024;
constexpr int kScanMaxBlocks = 2048;

// Inclusive scan of one value per thread across a 1024-thread block.
__device__ __forceinline__ int block_inclusive_scan(int v, int *s_wave /*[16]*/, int &block_total)
{
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        int o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    if (lane == 63) s_wave[wv] = v;
    __syncthreads();
    int wave_off = 0, total = 0;
    for (int i = 0; i < kScanThreads / 64; ++i) {
        int t = s_wave[i];
        if (i < wv) wave_off += t;
        total += t;
    }
    __syncthreads();
    block_total = total;
    return v + wave_off;
}

// PHASE 1: per-segment sums.  PHASE 3: exclusive offsets written back.
template <int PHASE>
__global__ __launch_bounds__(kScanThreads) void scan_segments_kernel(int *__restrict__ data, int n, int seg_len,
                                                                     int *__restrict__ sums)
{
    __shared__ int s_wave[kScanThreads / 64];
    const int seg_begin = blockIdx.x * seg_len;
    const int seg_end = min(seg_begin + seg_len, n);
    int running = (PHASE == 3) ? sums[blockIdx.x] : 0;
    for (int base = seg_begin; base < seg_end; base += kScanThreads) {
        const int i = base + threadIdx.x;
        int v = (i < seg_end) ? data[i] : 0;
        int total;
        int incl = block_inclusive_scan(v, s_wave, total);
        if (PHASE == 3 && i < seg_end) data[i] = running + incl - v;
        running += total;
    }
    if (PHASE == 1 && threadIdx.x == 0) sums[blockIdx.x] = running;
}

// PHASE 2: exclusive scan of the (<= 2048) segment sums in place.
__global__ __launch_bounds__(kScanThreads) void scan_sums_kernel(int *__restrict__ sums, int nseg)
{
    __shared__ int s_wave[kScanThreads / 64];
    int running = 0;
    for (int base = 0; base < nseg; base += kScanThreads) {
        const int i = base + threadIdx.x;
        int v = i < nseg ? sums[i] : 0;
        int total;
        int incl = block_inclusive_scan(v, s_wave, total);
        if (i < nseg) sums[i] = running + incl - v;
        running += total;
    }
}

// data[0..n) -> exclusive prefix sums; sums: int[2048] scratch.
int scan_exclusive_inplace(int *data, int n, int *sums, hipStream_t st)
{
    if (n <= 0) return MPS_OK;
    int nseg = (n + kScanThreads - 1) / kScanThreads;
    if (nseg > kScanMaxBlocks) nseg = kScanMaxBlocks;
    int seg_len = (n + nseg - 1) / nseg;
    seg_len = (seg_len + kScanThreads - 1) / kScanThreads * kScanThreads;
    nseg = (n + seg_len - 1) / seg_len;
    hipLaunchKernelGGL((scan_segments_kernel<1>), dim3(nseg), dim3(kScanThreads), 0, st, data, n, seg_len, sums);
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(kScanThreads), 0, st, sums, nseg);
    hipLaunchKernelGGL((scan_segments_kernel<3>), dim3(nseg), dim3(kScanThreads), 0, st, data, n, seg_len, sums);
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
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

template <typename T>
__global__ __launch_bounds__(256) void tile_gather_values_kernel(const T *__restrict__ val,
                                                                  const int *__restrict__ perm, int nnz,
                                                                  T *__restrict__ out)
{
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nnz) out[i] = val[perm[i]];
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
// Launch helpers
// ---------------------------------------------------------------------------
inline bool aligned_to(const void *p, unsigned a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// log2 of the row pitch in bytes when the fast addressing applies, else -1.
int pow2_row_shift(int n_rows, int K, int elem_bytes)
{
    uint64_t rb = (uint64_t)K * elem_bytes;
    if (rb & (rb - 1)) return -1;
    if ((uint64_t)(n_rows > 0 ? n_rows : 1) * rb >= (1ull << 32)) return -1;
    int sh = 0;
    while ((1ull << sh) < rb) ++sh;
    return sh;
}

struct SpmmShape {
    mps_lane_shape ls;
    int tpw;
    int num_waves;
    int row_shift;  // >= 0: power-of-two pitch, 32-bit offsets
};

int make_spmm_shape(int n_rows, int K, int P, int tpw, int elem_bytes, SpmmShape &sh)
{
    if (K < 1 || P < 1 || tpw < 0) return MPS_ERR_INVALID_ARG;
    sh.ls = mps_make_lane_shape(K, elem_bytes);
    if (tpw == 0) tpw = sh.ls.groups;
    if (tpw > sh.ls.groups) return MPS_ERR_TPW;
    sh.tpw = tpw;
    sh.num_waves = (P + tpw - 1) / tpw;
    sh.row_shift = pow2_row_shift(n_rows, K, elem_bytes);
    return MPS_OK;
}

size_t carry_bytes_for(int num_waves, int K)
{
    size_t rows = ((size_t)num_waves + 63) / 64 * 64;
    return rows * sizeof(int) + 2 * (size_t)num_waves * K * sizeof(float);
}

// Gathers in flight per lane between waits: tuning knob, 8 or 16.
int gather_batch()
{
    static int b = [] {
        const char *e = std::getenv("MPS_GATHER_BATCH");
        int v = e ? std::atoi(e) : 0;
        return v == 16 ? 16 : 8;
    }();
    return b;
}

template <typename T, typename TOut, int VEC>
int launch_spmm(const int *row_ptr, const int *col_idx, const T *val, const T *X, TOut *Y, int nnz, int K, int P,
                const int *cx, const int *cy, const SpmmShape &sh, void *ws, unsigned phases, hipStream_t st)
{
    const int W = sh.num_waves;
    size_t rows = ((size_t)W + 63) / 64 * 64;
    int *ws_head_row = static_cast<int *>(ws);
    float *ws_head = reinterpret_cast<float *>(ws_head_row + rows);
    float *ws_tail = ws_head + (size_t)W * K;
    if (phases & MPS_PHASE_MAIN) {
        dim3 grid((W + kWavesPerBlock - 1) / kWavesPerBlock, sh.ls.col_tiles);
#define MPS_LAUNCH_MAIN(POW2, BATCH)                                                                        \
    hipLaunchKernelGGL((mp_spmm_kernel<T, TOut, VEC, POW2, BATCH>), grid, dim3(kBlock), 0, st, row_ptr,     \
                       col_idx, val, X, Y, cx, cy, nnz, K, P, sh.ls.lanes_log2, sh.tpw, W, sh.row_shift,    \
                       ws_head_row, ws_head, ws_tail)
        if (sh.row_shift >= 0) {
            if (gather_batch() == 16) MPS_LAUNCH_MAIN(true, 16); else MPS_LAUNCH_MAIN(true, 8);
        } else {
            MPS_LAUNCH_MAIN(false, 8);
        }
#undef MPS_LAUNCH_MAIN
        MPS_HIP_TRY(hipGetLastError());
    }
    if (phases & MPS_PHASE_FIXUP) {
        long long threads = (long long)W * K;
        unsigned blocks = (unsigned)((threads + 255) / 256);
        hipLaunchKernelGGL((mp_fixup_kernel<TOut>), dim3(blocks), dim3(256), 0, st, ws_head_row, ws_head, ws_tail,
                           Y, W, K);
        MPS_HIP_TRY(hipGetLastError());
    }
    return MPS_OK;
}

template <typename T, typename TOut>
int launch_spmm_any(const int *row_ptr, const int *col_idx, const T *val, const T *X, TOut *Y, int nnz, int K,
                    int P, const int *cx, const int *cy, const SpmmShape &sh, void *ws, unsigned phases,
                    hipStream_t st)
{
    if (sh.ls.vec == 1)
        return launch_spmm<T, TOut, 1>(row_ptr, col_idx, val, X, Y, nnz, K, P, cx, cy, sh, ws, phases, st);
    return launch_spmm<T, TOut, 16 / (int)sizeof(T)>(row_ptr, col_idx, val, X, Y, nnz, K, P, cx, cy, sh, ws, phases,
                                                     st);
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
    return launch_spmm_any<T, T>(row_ptr, col_idx, val, X, Y, nnz, K, P, cx, cy, sh, ws, phases,
                                 static_cast<hipStream_t>(stream));
}

// Tiled: the main kernel writes fp32 partial rows for the num_slabs * n_rows
// virtual rows; the reduce kernel produces Y.
size_t tiled_part_bytes(int n_rows, int num_slabs, int K)
{
    size_t b = (size_t)num_slabs * (size_t)n_rows * K * sizeof(float);
    return (b + 255) / 256 * 256;
}

template <typename T>
int spmm_tiled_entry(const int *vrow_ptr, const int *col_t, const T *val_t, const T *X, T *Y, int n_rows, int nnz,
                     int K, int num_slabs, int P, const int *cx, const int *cy, int tpw, void *ws, size_t ws_bytes,
                     unsigned phases, void *stream)
{
    if (num_slabs < 1) return MPS_ERR_INVALID_ARG;
    const long long n_vrows = (long long)num_slabs * n_rows;
    int rc = check_spmm_args<T>(vrow_ptr, col_t, val_t, X, Y, n_rows, n_vrows, nnz, K, P, cx, cy);
    if (rc != MPS_OK) return rc;
    SpmmShape sh;
    rc = make_spmm_shape(n_rows, K, P, tpw, (int)sizeof(T), sh);
    if (rc != MPS_OK) return rc;
    const size_t part_b = tiled_part_bytes(n_rows, num_slabs, K);
    if (!ws || ws_bytes < part_b + carry_bytes_for(sh.num_waves, K)) return MPS_ERR_WORKSPACE;
    if (!aligned_to(ws, 16)) return MPS_ERR_ALIGNMENT;
    if (n_rows == 0) return MPS_OK;
    float *part = static_cast<float *>(ws);
    void *carry = static_cast<char *>(ws) + part_b;
    hipStream_t st = static_cast<hipStream_t>(stream);
    rc = launch_spmm_any<T, float>(vrow_ptr, col_t, val_t, X, part, nnz, K, P, cx, cy, sh, carry, phases, st);
    if (rc != MPS_OK) return rc;
    if (phases & MPS_PHASE_REDUCE) {
        const size_t per_slab = (size_t)n_rows * K;
        if (K % 4 == 0) {
            unsigned blocks = (unsigned)((per_slab / 4 + 255) / 256);
            hipLaunchKernelGGL((tile_reduce_kernel<T, 4>), dim3(blocks), dim3(256), 0, st, part, Y, n_rows, K,
                               num_slabs);
        } else {
            unsigned blocks = (unsigned)((per_slab + 255) / 256);
            hipLaunchKernelGGL((tile_reduce_kernel<T, 1>), dim3(blocks), dim3(256), 0, st, part, Y, n_rows, K,
                               num_slabs);
        }
        MPS_HIP_TRY(hipGetLastError());
    }
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

// ---- column-slab tiling ---------------------------------------------------

int mps_tile_shape(int n_rows, int nnz, int K, int elem_bytes, size_t slab_bytes, int *num_slabs_out,
                   int *slab_cols_out)
{
    if (!num_slabs_out || !slab_cols_out || n_rows < 0 || nnz < 0 || K < 1) return MPS_ERR_INVALID_ARG;
    if (elem_bytes != 4 && elem_bytes != 2) return MPS_ERR_INVALID_ARG;
    if (slab_bytes == 0) slab_bytes = 2u << 20;
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

int mps_tile_build(const int *d_row_ptr, const int *d_col_idx, int n_rows, int nnz, int num_slabs,
                   int slab_cols, int *d_vrow_ptr, int *d_col_tiled, int *d_perm, int *d_scratch, void *stream)
{
    if (!d_row_ptr || !d_vrow_ptr || !d_scratch || n_rows < 0 || nnz < 0) return MPS_ERR_INVALID_ARG;
    if (num_slabs < 1 || slab_cols < 1) return MPS_ERR_INVALID_ARG;
    if (nnz > 0 && (!d_col_idx || !d_col_tiled || !d_perm)) return MPS_ERR_INVALID_ARG;
    if ((long long)num_slabs * slab_cols < n_rows) return MPS_ERR_INVALID_ARG;
    const long long nv = (long long)num_slabs * n_rows;
    if (nv + 1 + nnz > INT_MAX) return MPS_ERR_UNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int *first = d_scratch;           // [nv]
    int *sums = d_scratch + nv;       // [2048]
    int *bad = sums + kScanMaxBlocks; // [1]
    int zero = 0, h_bad = 0;
    MPS_HIP_TRY(hipMemcpyAsync(bad, &zero, sizeof(int), hipMemcpyHostToDevice, st));
    if (nnz > 1) {
        unsigned blocks = (unsigned)(((long long)nnz + 255) / 256);
        hipLaunchKernelGGL(tile_sorted_check_kernel, dim3(blocks), dim3(256), 0, st, d_row_ptr, d_col_idx, n_rows,
                           nnz, bad);
    }
    {
        unsigned blocks = (unsigned)((nv + 1 + 255) / 256);
        hipLaunchKernelGGL(tile_count_kernel, dim3(blocks), dim3(256), 0, st, d_row_ptr, d_col_idx, n_rows,
                           num_slabs, slab_cols, first, d_vrow_ptr);
    }
    MPS_HIP_TRY(hipGetLastError());
    int rc = scan_exclusive_inplace(d_vrow_ptr, (int)nv + 1, sums, st);
    if (rc != MPS_OK) return rc;
    if (nnz > 0) {
        unsigned blocks = (unsigned)(((long long)nnz + 255) / 256);
        hipLaunchKernelGGL(tile_scatter_kernel, dim3(blocks), dim3(256), 0, st, d_row_ptr, d_col_idx, n_rows, nnz,
                           num_slabs, slab_cols, first, d_vrow_ptr, d_col_tiled, d_perm);
        MPS_HIP_TRY(hipGetLastError());
    }
    MPS_HIP_TRY(hipMemcpyAsync(&h_bad, bad, sizeof(int), hipMemcpyDeviceToHost, st));
    MPS_HIP_TRY(hipStreamSynchronize(st));
    return h_bad ? MPS_ERR_UNSORTED : MPS_OK;
}

int mps_tile_gather_values(const void *d_val, const int *d_perm, int nnz, int elem_bytes, void *d_val_tiled,
                           void *stream)
{
    if (nnz < 0 || (elem_bytes != 4 && elem_bytes != 2)) return MPS_ERR_INVALID_ARG;
    if (nnz == 0) return MPS_OK;
    if (!d_val || !d_perm || !d_val_tiled) return MPS_ERR_INVALID_ARG;
    unsigned blocks = (unsigned)(((long long)nnz + 255) / 256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (elem_bytes == 4)
        hipLaunchKernelGGL((tile_gather_values_kernel<float>), dim3(blocks), dim3(256), 0, st,
                           static_cast<const float *>(d_val), d_perm, nnz, static_cast<float *>(d_val_tiled));
    else
        hipLaunchKernelGGL((tile_gather_values_kernel<half_t>), dim3(blocks), dim3(256), 0, st,
                           static_cast<const half_t *>(d_val), d_perm, nnz, static_cast<half_t *>(d_val_tiled));
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

int mps_spmm_tiled_workspace_bytes(int n_rows, int num_slabs, int P, int K, int tpw, int elem_bytes,
                                   size_t *bytes_out)
{
    if (!bytes_out || n_rows < 0 || num_slabs < 1 || (elem_bytes != 4 && elem_bytes != 2))
        return MPS_ERR_INVALID_ARG;
    SpmmShape sh;
    int rc = make_spmm_shape(n_rows, K, P, tpw, elem_bytes, sh);
    if (rc != MPS_OK) return rc;
    *bytes_out = tiled_part_bytes(n_rows, num_slabs, K) + carry_bytes_for(sh.num_waves, K);
    return MPS_OK;
}

int mps_spmm_tiled_f32_phases(const int *d_vrow_ptr, const int *d_col_tiled, const float *d_val_tiled,
                              const float *d_X, float *d_Y, int n_rows, int nnz, int K, int num_slabs, int P,
                              const int *d_coord_x, const int *d_coord_y, int tpw, void *d_workspace,
                              size_t workspace_bytes, unsigned phases, void *stream)
{
    return spmm_tiled_entry<float>(d_vrow_ptr, d_col_tiled, d_val_tiled, d_X, d_Y, n_rows, nnz, K, num_slabs, P,
                                   d_coord_x, d_coord_y, tpw, d_workspace, workspace_bytes, phases, stream);
}

int mps_spmm_tiled_f32(const int *d_vrow_ptr, const int *d_col_tiled, const float *d_val_tiled, const float *d_X,
                       float *d_Y, int n_rows, int nnz, int K, int num_slabs, int P, const int *d_coord_x,
                       const int *d_coord_y, int tpw, void *d_workspace, size_t workspace_bytes, void *stream)
{
    return spmm_tiled_entry<float>(d_vrow_ptr, d_col_tiled, d_val_tiled, d_X, d_Y, n_rows, nnz, K, num_slabs, P,
                                   d_coord_x, d_coord_y, tpw, d_workspace, workspace_bytes,
                                   MPS_PHASE_MAIN | MPS_PHASE_FIXUP | MPS_PHASE_REDUCE, stream);
}

int mps_spmm_tiled_f16_phases(const int *d_vrow_ptr, const int *d_col_tiled, const uint16_t *d_val_tiled,
                              const uint16_t *d_X, uint16_t *d_Y, int n_rows, int nnz, int K, int num_slabs,
                              int P, const int *d_coord_x, const int *d_coord_y, int tpw, void *d_workspace,
                              size_t workspace_bytes, unsigned phases, void *stream)
{
    return spmm_tiled_entry<half_t>(d_vrow_ptr, d_col_tiled, reinterpret_cast<const half_t *>(d_val_tiled),
                                    reinterpret_cast<const half_t *>(d_X), reinterpret_cast<half_t *>(d_Y), n_rows,
                                    nnz, K, num_slabs, P, d_coord_x, d_coord_y, tpw, d_workspace, workspace_bytes,
                                    phases, stream);
}

int mps_spmm_tiled_f16(const int *d_vrow_ptr, const int *d_col_tiled, const uint16_t *d_val_tiled,
                       const uint16_t *d_X, uint16_t *d_Y, int n_rows, int nnz, int K, int num_slabs, int P,
                       const int *d_coord_x, const int *d_coord_y, int tpw, void *d_workspace,
                       size_t workspace_bytes, void *stream)
{
    return mps_spmm_tiled_f16_phases(d_vrow_ptr, d_col_tiled, d_val_tiled, d_X, d_Y, n_rows, nnz, K, num_slabs, P,
                                     d_coord_x, d_coord_y, tpw, d_workspace, workspace_bytes,
                                     MPS_PHASE_MAIN | MPS_PHASE_FIXUP | MPS_PHASE_REDUCE, stream);
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
    hipLaunchKernelGGL((rowwise_spmm_kernel<float, VEC, POW2, 8>), grid, dim3(kBlock), 0, st, d_row_ptr,  \
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
    hipLaunchKernelGGL((nzsplit_spmm_kernel<float, VEC, POW2, 8>), grid, dim3(kBlock), 0, st, d_col_idx, \
                       d_val, d_X, d_Y, nnz, K, ls.lanes_log2, row_shift, d_part_ptr, d_part2node,       \
                       num_parts, num_waves)
    if (ls.vec == 4) { if (row_shift >= 0) MPS_LAUNCH_NZSPLIT(4, true); else MPS_LAUNCH_NZSPLIT(4, false); }
    else { if (row_shift >= 0) MPS_LAUNCH_NZSPLIT(1, true); else MPS_LAUNCH_NZSPLIT(1, false); }
#undef MPS_LAUNCH_NZSPLIT
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

}  // extern "C"
