// Device half of the MergePath-SpMM C ABI: hand-written HIP kernels for
// gfx950 (CDNA4, 64-lane wavefronts) and their launchers.
//
// Work decomposition.  A wavefront is cut into lane-groups of L = 4..64 lanes
// (L * VEC >= min(K, 64 * VEC) columns, VEC = one 16-byte load per lane where
// K allows).  In the merge-path kernel every lane-group walks one partition
// of the reference schedule (src/MergePathSpMM.cu:300-385): `cost` merge
// items = row ends + nonzeros.  The group streams its col_idx / val run
// through LDS in 16-nonzero windows (one coalesced 64-byte load per array per
// window), gathers the 16 dense rows with 16-byte loads, and accumulates in
// fp32 registers.  Rows that end inside a partition after its first row end
// are stored directly.  A group's first finished row and its unfinished last
// row are partial: they are first combined across the groups of the
// wavefront through LDS, and what still crosses the wavefront boundary is
// written to a carry-out record that a second kernel folds in.  No atomics.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>

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
// Per-(element type, vector width) access to the dense matrices.
// ---------------------------------------------------------------------------
template <typename T, int VEC>
struct XOps;

template <>
struct XOps<float, 4> {
    using Raw = float4;
    static __device__ __forceinline__ Raw zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    static __device__ __forceinline__ void fma(float (&acc)[4], float v, const Raw &r)
    {
        acc[0] = __builtin_fmaf(v, r.x, acc[0]);
        acc[1] = __builtin_fmaf(v, r.y, acc[1]);
        acc[2] = __builtin_fmaf(v, r.z, acc[2]);
        acc[3] = __builtin_fmaf(v, r.w, acc[3]);
    }
    static __device__ __forceinline__ void store(float *p, const float (&acc)[4])
    {
        *reinterpret_cast<float4 *>(p) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    }
};

template <>
struct XOps<float, 1> {
    using Raw = float;
    static __device__ __forceinline__ Raw zero() { return 0.f; }
    static __device__ __forceinline__ void fma(float (&acc)[1], float v, const Raw &r)
    {
        acc[0] = __builtin_fmaf(v, r, acc[0]);
    }
    static __device__ __forceinline__ void store(float *p, const float (&acc)[1]) { *p = acc[0]; }
};

typedef half_t half8_t __attribute__((ext_vector_type(8)));

template <>
struct XOps<half_t, 8> {
    using Raw = half8_t;
    static __device__ __forceinline__ Raw zero() { return Raw{0, 0, 0, 0, 0, 0, 0, 0}; }
    static __device__ __forceinline__ void fma(float (&acc)[8], float v, const Raw &r)
    {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(v, (float)r[i], acc[i]);
    }
    static __device__ __forceinline__ void store(half_t *p, const float (&acc)[8])
    {
        Raw o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (half_t)acc[i];
        *reinterpret_cast<Raw *>(p) = o;
    }
};

template <>
struct XOps<half_t, 1> {
    using Raw = half_t;
    static __device__ __forceinline__ Raw zero() { return (half_t)0; }
    static __device__ __forceinline__ void fma(float (&acc)[1], float v, const Raw &r)
    {
        acc[0] = __builtin_fmaf(v, (float)r, acc[0]);
    }
    static __device__ __forceinline__ void store(half_t *p, const float (&acc)[1]) { *p = (half_t)acc[0]; }
};

template <bool WIDE>
struct OffT {
    using type = unsigned;
};
template <>
struct OffT<true> {
    using type = size_t;
};

// Four consecutive values (16-byte aligned for fp32, 8-byte for fp16) -> fp32.
__device__ __forceinline__ float4 load_val4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 load_val4(const half_t *p)
{
    typedef half_t half4_t __attribute__((ext_vector_type(4)));
    half4_t h = *reinterpret_cast<const half4_t *>(p);
    return make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
}

// Stage the window [wbase, wbase + 16) of a lane-group's col_idx / val run
// into its LDS slot: lanes 0..3 of the group each move 4 nonzeros.
template <typename T>
__device__ __forceinline__ void stage_window(const int *__restrict__ col_idx, const T *__restrict__ val,
                                             int nnz, int wbase, int s, int *s_col, float *s_val)
{
    if (s < 4) {
        int i0 = wbase + 4 * s;
        int4 c = make_int4(0, 0, 0, 0);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i0 + 3 < nnz) {
            c = *reinterpret_cast<const int4 *>(col_idx + i0);
            v = load_val4(val + i0);
        } else {
            if (i0 + 0 < nnz) { c.x = col_idx[i0 + 0]; v.x = (float)val[i0 + 0]; }
            if (i0 + 1 < nnz) { c.y = col_idx[i0 + 1]; v.y = (float)val[i0 + 1]; }
            if (i0 + 2 < nnz) { c.z = col_idx[i0 + 2]; v.z = (float)val[i0 + 2]; }
        }
        *reinterpret_cast<int4 *>(s_col + 4 * s) = c;
        *reinterpret_cast<float4 *>(s_val + 4 * s) = v;
    }
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
template <typename T, int VEC, bool WIDE, int BATCH>
__global__ __launch_bounds__(kBlock) void mp_spmm_kernel(
    const int *__restrict__ row_ptr, const int *__restrict__ col_idx, const T *__restrict__ val,
    const T *__restrict__ X, T *__restrict__ Y, const int *__restrict__ coord_x,
    const int *__restrict__ coord_y, int nnz, int K, int P, int lanes_log2, int tpw, int num_waves,
    int *__restrict__ ws_head_row, float *__restrict__ ws_head, float *__restrict__ ws_tail)
{
    using XO = XOps<T, VEC>;
    using Raw = typename XO::Raw;
    using off_t_ = typename OffT<WIDE>::type;
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
    const off_t_ row_bytes = (off_t_)K * (off_t_)sizeof(T);
    const off_t_ col_byte = (off_t_)kcol * (off_t_)sizeof(T);
    const char *xb = reinterpret_cast<const char *>(X);

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
    int row_end = (x < x_end) ? row_ptr[x] : INT_MAX;

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
            XO::store(Y + (size_t)row * K + kcol, acc);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        ++x;
        row_end = (x < x_end) ? row_ptr[x] : INT_MAX;
    };

    int wbase = y_begin & ~3;
    while (__any(wbase < y_end)) {
        if (wbase < y_end) stage_window<T>(col_idx, val, nnz, wbase, s, s_col, s_val);
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
            for (int j = 0; j < BATCH; ++j) {
                const int idx = wbase + b + j;
                const bool ok = col_ok && idx >= y_begin && idx < y_end;
                xr[j] = XO::zero();
                if (ok) xr[j] = *reinterpret_cast<const Raw *>(xb + ((off_t_)cols[j] * row_bytes + col_byte));
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int idx = wbase + b + j;
                if (idx >= y_begin && idx < y_end) {
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
                    Y[(size_t)hr * K + kc] = (T)v;
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
template <typename T>
__global__ __launch_bounds__(256) void mp_fixup_kernel(const int *__restrict__ ws_head_row,
                                                        const float *__restrict__ ws_head,
                                                        const float *__restrict__ ws_tail,
                                                        T *__restrict__ Y, int num_waves, int K)
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
    Y[(size_t)hr * K + k] = (T)sum;
}

// ---------------------------------------------------------------------------
// One lane-group accumulates the nonzero range [y_begin, y_end) of one row.
// Wave-uniform control flow: every group of the wave runs the same number of
// rounds, idle ones with an empty range.
// ---------------------------------------------------------------------------
template <typename T, int VEC, bool WIDE, int BATCH>
__device__ __forceinline__ void accumulate_range(const int *__restrict__ col_idx,
                                                 const T *__restrict__ val, const char *xb, int nnz,
                                                 int y_begin, int y_end, bool col_ok,
                                                 typename OffT<WIDE>::type row_bytes,
                                                 typename OffT<WIDE>::type col_byte, int s, int *s_col,
                                                 float *s_val, float (&acc)[VEC])
{
    using XO = XOps<T, VEC>;
    using Raw = typename XO::Raw;
    using off_t_ = typename OffT<WIDE>::type;
    int wbase = y_begin & ~3;
    while (__any(wbase < y_end)) {
        if (wbase < y_end) stage_window<T>(col_idx, val, nnz, wbase, s, s_col, s_val);
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
            for (int j = 0; j < BATCH; ++j) {
                const int idx = wbase + b + j;
                const bool ok = col_ok && idx >= y_begin && idx < y_end;
                xr[j] = XO::zero();
                if (ok) xr[j] = *reinterpret_cast<const Raw *>(xb + ((off_t_)cols[j] * row_bytes + col_byte));
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                const int idx = wbase + b + j;
                if (idx >= y_begin && idx < y_end) XO::fma(acc, vals[j], xr[j]);
            }
        }
        wbase += kWindow;
        wave_lds_sync();
    }
}

// Row-wise comparison kernel (src/row_wise.cu:194-240): wavefront w owns the
// rows [int(step * w), int(step * (w + 1))); its lane-groups take those rows
// round-robin, one whole row per group, plain stores.
template <typename T, int VEC, bool WIDE, int BATCH>
__global__ __launch_bounds__(kBlock) void rowwise_spmm_kernel(
    const int *__restrict__ row_ptr, const int *__restrict__ col_idx, const T *__restrict__ val,
    const T *__restrict__ X, T *__restrict__ Y, int n_rows, int nnz, int K, int lanes_log2,
    int num_waves, float step)
{
    using XO = XOps<T, VEC>;
    using off_t_ = typename OffT<WIDE>::type;
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
    const off_t_ row_bytes = (off_t_)K * (off_t_)sizeof(T);
    const off_t_ col_byte = (off_t_)kcol * (off_t_)sizeof(T);
    const char *xb = reinterpret_cast<const char *>(X);
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
        accumulate_range<T, VEC, WIDE, BATCH>(col_idx, val, xb, nnz, y_begin, y_end, col_ok, row_bytes,
                                               col_byte, s, s_col, s_val, acc);
        if (row_ok && col_ok) XO::store(Y + (size_t)row * K + kcol, acc);
    }
}

// Nonzero-splitting comparison kernel (src/nz_splitting.cu:318-445): one
// group of at most part_size nonzeros per lane-group, ending in atomic adds.
template <typename T, int VEC, bool WIDE, int BATCH>
__global__ __launch_bounds__(kBlock) void nzsplit_spmm_kernel(
    const int *__restrict__ col_idx, const T *__restrict__ val, const T *__restrict__ X,
    float *__restrict__ Y, int nnz, int K, int lanes_log2, const int *__restrict__ part_ptr,
    const int *__restrict__ part2node, int num_parts, int num_waves)
{
    using off_t_ = typename OffT<WIDE>::type;
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
    const off_t_ row_bytes = (off_t_)K * (off_t_)sizeof(T);
    const off_t_ col_byte = (off_t_)kcol * (off_t_)sizeof(T);
    const char *xb = reinterpret_cast<const char *>(X);
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
    accumulate_range<T, VEC, WIDE, BATCH>(col_idx, val, xb, nnz, y_begin, y_end, col_ok, row_bytes,
                                           col_byte, s, s_col, s_val, acc);
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
constexpr int kScanThreads = 1024;
constexpr int kScanMaxBlocks = 2048;

__device__ __forceinline__ int parts_of_row(const int *__restrict__ row_ptr, int r, int n_rows,
                                            int part_size)
{
    if (r >= n_rows) return 0;
    int degree = row_ptr[r + 1] - row_ptr[r];
    return degree / part_size + (degree % part_size != 0);
}

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

// phase 1: per-segment sums; phase 3: exclusive offsets written to out[0..n].
template <int PHASE>
__global__ __launch_bounds__(kScanThreads) void nzsplit_scan_kernel(const int *__restrict__ row_ptr,
                                                                    int n_rows, int part_size,
                                                                    int seg_len, int *__restrict__ sums,
                                                                    int *__restrict__ out)
{
    __shared__ int s_wave[kScanThreads / 64];
    const int seg_begin = blockIdx.x * seg_len;
    const int seg_end = min(seg_begin + seg_len, n_rows + 1);
    int running = (PHASE == 3) ? sums[blockIdx.x] : 0;
    for (int base = seg_begin; base < seg_end; base += kScanThreads) {
        const int r = base + threadIdx.x;
        int v = (r < seg_end) ? parts_of_row(row_ptr, r, n_rows, part_size) : 0;
        int total;
        int incl = block_inclusive_scan(v, s_wave, total);
        if (PHASE == 3 && r < seg_end) out[r] = running + incl - v;
        running += total;
    }
    if (PHASE == 1 && threadIdx.x == 0) sums[blockIdx.x] = running;
}

// phase 2: exclusive scan of the (<= 2048) segment sums in place.
__global__ __launch_bounds__(kScanThreads) void nzsplit_scan_sums_kernel(int *__restrict__ sums, int nseg)
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
// Launch helpers
// ---------------------------------------------------------------------------
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

struct SpmmShape {
    mps_lane_shape ls;
    int tpw;
    int num_waves;
    bool wide;
};

int make_spmm_shape(int n_rows, int K, int P, int tpw, int elem_bytes, SpmmShape &sh)
{
    if (K < 1 || P < 1 || tpw < 0) return MPS_ERR_INVALID_ARG;
    sh.ls = mps_make_lane_shape(K, elem_bytes);
    if (tpw == 0) tpw = sh.ls.groups;
    if (tpw > sh.ls.groups) return MPS_ERR_TPW;
    sh.tpw = tpw;
    sh.num_waves = (P + tpw - 1) / tpw;
    sh.wide = (uint64_t)(n_rows > 0 ? n_rows : 1) * (uint64_t)K * (uint64_t)elem_bytes >= (1ull << 32);
    return MPS_OK;
}

size_t workspace_bytes_for(int num_waves, int K)
{
    size_t rows = ((size_t)num_waves + 63) / 64 * 64;
    return rows * sizeof(int) + 2 * (size_t)num_waves * K * sizeof(float);
}

constexpr int kBatch = 8;

template <typename T, int VEC>
int launch_spmm(const int *row_ptr, const int *col_idx, const T *val, const T *X, T *Y, int n_rows,
                int nnz, int K, int P, const int *cx, const int *cy, const SpmmShape &sh, void *ws,
                unsigned phases, hipStream_t st)
{
    (void)n_rows;
    const int W = sh.num_waves;
    size_t rows = ((size_t)W + 63) / 64 * 64;
    int *ws_head_row = static_cast<int *>(ws);
    float *ws_head = reinterpret_cast<float *>(ws_head_row + rows);
    float *ws_tail = ws_head + (size_t)W * K;
    if (phases & MPS_PHASE_MAIN) {
        dim3 grid((W + kWavesPerBlock - 1) / kWavesPerBlock, sh.ls.col_tiles);
        if (sh.wide)
            hipLaunchKernelGGL((mp_spmm_kernel<T, VEC, true, kBatch>), grid, dim3(kBlock), 0, st, row_ptr,
                               col_idx, val, X, Y, cx, cy, nnz, K, P, sh.ls.lanes_log2, sh.tpw, W,
                               ws_head_row, ws_head, ws_tail);
        else
            hipLaunchKernelGGL((mp_spmm_kernel<T, VEC, false, kBatch>), grid, dim3(kBlock), 0, st, row_ptr,
                               col_idx, val, X, Y, cx, cy, nnz, K, P, sh.ls.lanes_log2, sh.tpw, W,
                               ws_head_row, ws_head, ws_tail);
        MPS_HIP_TRY(hipGetLastError());
    }
    if (phases & MPS_PHASE_FIXUP) {
        long long threads = (long long)W * K;
        unsigned blocks = (unsigned)((threads + 255) / 256);
        hipLaunchKernelGGL((mp_fixup_kernel<T>), dim3(blocks), dim3(256), 0, st, ws_head_row, ws_head,
                           ws_tail, Y, W, K);
        MPS_HIP_TRY(hipGetLastError());
    }
    return MPS_OK;
}

template <typename T>
int spmm_entry(const int *row_ptr, const int *col_idx, const T *val, const T *X, T *Y, int n_rows,
               int nnz, int K, int P, const int *cx, const int *cy, int tpw, void *ws, size_t ws_bytes,
               unsigned phases, void *stream)
{
    if (n_rows < 0 || nnz < 0 || K < 1 || P < 1) return MPS_ERR_INVALID_ARG;
    if (!row_ptr || !cx || !cy || (nnz > 0 && (!col_idx || !val))) return MPS_ERR_INVALID_ARG;
    if (n_rows > 0 && (!X || !Y)) return MPS_ERR_INVALID_ARG;
    if ((long long)n_rows + 1 + nnz > INT_MAX) return MPS_ERR_UNSUPPORTED;
    if ((long long)P > INT_MAX / 2) return MPS_ERR_UNSUPPORTED;
    if (!aligned16(col_idx) || !aligned16(val) || !aligned16(X) || !aligned16(Y)) return MPS_ERR_ALIGNMENT;
    SpmmShape sh;
    int rc = make_spmm_shape(n_rows, K, P, tpw, (int)sizeof(T), sh);
    if (rc != MPS_OK) return rc;
    if ((long long)sh.num_waves * K > (1ll << 40)) return MPS_ERR_UNSUPPORTED;
    if (!ws || ws_bytes < workspace_bytes_for(sh.num_waves, K)) return MPS_ERR_WORKSPACE;
    if (!aligned16(ws)) return MPS_ERR_ALIGNMENT;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (sh.ls.vec == 1)
        return launch_spmm<T, 1>(row_ptr, col_idx, val, X, Y, n_rows, nnz, K, P, cx, cy, sh, ws, phases, st);
    return launch_spmm<T, 16 / (int)sizeof(T)>(row_ptr, col_idx, val, X, Y, n_rows, nnz, K, P, cx, cy, sh,
                                               ws, phases, st);
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
    *bytes_out = workspace_bytes_for(sh.num_waves, K);
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
    if (!aligned16(d_col_idx) || !aligned16(d_val) || !aligned16(d_X) || !aligned16(d_Y))
        return MPS_ERR_ALIGNMENT;
    if (n_rows == 0) return MPS_OK;
    mps_lane_shape ls = mps_make_lane_shape(K, 4);
    bool wide = (uint64_t)n_rows * (uint64_t)K * 4ull >= (1ull << 32);
    float step = (float)n_rows / (float)num_waves;
    dim3 grid((num_waves + kWavesPerBlock - 1) / kWavesPerBlock, ls.col_tiles);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define MPS_LAUNCH_ROWWISE(VEC, WIDE)                                                                    \
    hipLaunchKernelGGL((rowwise_spmm_kernel<float, VEC, WIDE, kBatch>), grid, dim3(kBlock), 0, st,       \
                       d_row_ptr, d_col_idx, d_val, d_X, d_Y, n_rows, nnz, K, ls.lanes_log2, num_waves,   \
                       step)
    if (ls.vec == 4) { if (wide) MPS_LAUNCH_ROWWISE(4, true); else MPS_LAUNCH_ROWWISE(4, false); }
    else { if (wide) MPS_LAUNCH_ROWWISE(1, true); else MPS_LAUNCH_ROWWISE(1, false); }
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
    int nseg = (n + kScanThreads - 1) / kScanThreads;
    if (nseg > kScanMaxBlocks) nseg = kScanMaxBlocks;
    int seg_len = (n + nseg - 1) / nseg;
    seg_len = (seg_len + kScanThreads - 1) / kScanThreads * kScanThreads;
    nseg = (n + seg_len - 1) / seg_len;
    int *offsets = d_scratch;          // [n_rows + 1]
    int *sums = d_scratch + n;         // [<= 2048]
    hipLaunchKernelGGL((nzsplit_scan_kernel<1>), dim3(nseg), dim3(kScanThreads), 0, st, d_row_ptr, n_rows,
                       part_size, seg_len, sums, offsets);
    hipLaunchKernelGGL(nzsplit_scan_sums_kernel, dim3(1), dim3(kScanThreads), 0, st, sums, nseg);
    hipLaunchKernelGGL((nzsplit_scan_kernel<3>), dim3(nseg), dim3(kScanThreads), 0, st, d_row_ptr, n_rows,
                       part_size, seg_len, sums, offsets);
    MPS_HIP_TRY(hipGetLastError());
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
    if (!aligned16(d_col_idx) || !aligned16(d_val) || !aligned16(d_X) || !aligned16(d_Y))
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
    bool wide = (uint64_t)n_rows * (uint64_t)K * 4ull >= (1ull << 32);
    int num_waves = (num_parts + ls.groups - 1) / ls.groups;
    dim3 grid((num_waves + kWavesPerBlock - 1) / kWavesPerBlock, ls.col_tiles);
#define MPS_LAUNCH_NZSPLIT(VEC, WIDE)                                                                  \
    hipLaunchKernelGGL((nzsplit_spmm_kernel<float, VEC, WIDE, kBatch>), grid, dim3(kBlock), 0, st,     \
                       d_col_idx, d_val, d_X, d_Y, nnz, K, ls.lanes_log2, d_part_ptr, d_part2node,     \
                       num_parts, num_waves)
    if (ls.vec == 4) { if (wide) MPS_LAUNCH_NZSPLIT(4, true); else MPS_LAUNCH_NZSPLIT(4, false); }
    else { if (wide) MPS_LAUNCH_NZSPLIT(1, true); else MPS_LAUNCH_NZSPLIT(1, false); }
#undef MPS_LAUNCH_NZSPLIT
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

}  // extern "C"
