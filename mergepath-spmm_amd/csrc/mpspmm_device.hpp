// Device code shared by the two halves of the library's GPU side
// (mpspmm_kernels.hip: the CSR entry points; mpspmm_plan.hip: plans).
// Everything lives in an anonymous namespace: each translation unit gets its
// own copy of the kernels it launches.
#ifndef MPSPMM_DEVICE_HPP
#define MPSPMM_DEVICE_HPP

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
constexpr int kXcds = 8;     // accelerator dies of an MI355X, each with its own L2
constexpr int kHotRoundsPerLoad = 1;    // rounds of the sliced arrays a hot wavefront loads at a time
constexpr int kHotWavesPerBlock = 16;   // workgroup of the LDS-resident ("hot") launch of a plan

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
struct XOps<half_t, 4> {
    using Raw = half4_t;
    static __device__ __forceinline__ void fma(float (&acc)[4], float v, const Raw &r)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_fmaf(v, (float)r[i], acc[i]);
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
// where the width allows.  Non-temporal (NT): output rows are written once and
// not read again by the kernel, so they should not displace X in L2.  The hot
// launch of a plan has no X in L2 to protect and waits less on plain stores
// (a load that follows a store in program order also waits for the store).
template <int VEC, bool NT = true>
__device__ __forceinline__ void store_acc(float *p, const float (&acc)[VEC])
{
    typedef float f4_t __attribute__((ext_vector_type(4)));
    if constexpr (VEC % 4 == 0) {
#pragma unroll
        for (int i = 0; i < VEC; i += 4) {
            f4_t v = {acc[i], acc[i + 1], acc[i + 2], acc[i + 3]};
            if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<f4_t *>(p + i));
            else *reinterpret_cast<f4_t *>(p + i) = v;
        }
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) __builtin_nontemporal_store(acc[i], p + i);
    }
}
template <int VEC, bool NT = true>
__device__ __forceinline__ void store_acc(half_t *p, const float (&acc)[VEC])
{
    if constexpr (VEC == 8) {
        half8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (half_t)acc[i];
        __builtin_nontemporal_store(o, reinterpret_cast<half8_t *>(p));
    } else if constexpr (VEC == 4) {
        half4_t o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = (half_t)acc[i];
        __builtin_nontemporal_store(o, reinterpret_cast<half4_t *>(p));
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) __builtin_nontemporal_store((half_t)acc[i], p + i);
    }
}

// A row piece of X read through a buffer descriptor, with or without the streaming hint (AUX bit 1,
// "nt": the line is the first to leave the caches again).  Two plain global loads on the two sides of
// a branch get folded into one by the compiler, which then drops the hint; buffer loads that differ
// in their cache-policy operand stay two instructions.
template <typename Raw, int AUX>
__device__ __forceinline__ Raw buffer_load_raw(__amdgpu_buffer_rsrc_t rsrc, unsigned off)
{
    if constexpr (sizeof(Raw) == 16) {
        return __builtin_bit_cast(Raw, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, AUX));
    } else if constexpr (sizeof(Raw) == 8) {
        return __builtin_bit_cast(Raw, __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)off, 0, AUX));
    } else if constexpr (sizeof(Raw) == 4) {
        return __builtin_bit_cast(Raw, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)off, 0, AUX));
    } else {
        static_assert(sizeof(Raw) == 2, "rows of X are read 2, 4, 8 or 16 bytes at a time");
        return __builtin_bit_cast(Raw, __builtin_amdgcn_raw_buffer_load_b16(rsrc, (int)off, 0, AUX));
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
    // POW2 only: row c with the streaming hint (streamed) or without, through the buffer descriptor of X
    __device__ __forceinline__ Raw load_hinted(__amdgpu_buffer_rsrc_t rsrc, int c, bool streamed) const
    {
        static_assert(POW2, "32-bit offsets");
        const unsigned off = ((unsigned)c << row_shift) | col_byte;
        return streamed ? buffer_load_raw<Raw, 2>(rsrc, off) : buffer_load_raw<Raw, 0>(rsrc, off);
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


// Elements [e0, e0 + 4) of a plan's sliced arrays: 16-byte aligned, padded to
// whole round blocks, so no bounds are needed.
__device__ __forceinline__ Win load_slice_vals(const float *p, Win w)
{
    typedef float f4_t __attribute__((ext_vector_type(4)));
    f4_t t = __builtin_nontemporal_load(reinterpret_cast<const f4_t *>(p));
    w.v = make_float4(t[0], t[1], t[2], t[3]);
    return w;
}
__device__ __forceinline__ Win load_slice_vals(const half_t *p, Win w)
{
    half4_t h = __builtin_nontemporal_load(reinterpret_cast<const half4_t *>(p));
    w.v = make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
    return w;
}
__device__ __forceinline__ int4 load_slice_cols(const int *__restrict__ cols, size_t e0)
{
    typedef int i4_t __attribute__((ext_vector_type(4)));
    i4_t t = __builtin_nontemporal_load(reinterpret_cast<const i4_t *>(cols + e0));
    return make_int4(t[0], t[1], t[2], t[3]);
}
template <typename T>
__device__ __forceinline__ Win load_slice(const int *__restrict__ cols, const T *__restrict__ vals, size_t e0)
{
    Win w;
    w.c = load_slice_cols(cols, e0);
    return load_slice_vals(vals + e0, w);
}

// ---------------------------------------------------------------------------
// Merge-path SpMM, main kernel.
// ---------------------------------------------------------------------------
//
// SLICED = false: col_idx / val are the CSR arrays; every lane-group stages
//   its own 16-nonzero windows (two 64-byte loads per window).
// SLICED = true: col_idx / val are the sliced arrays of a plan: the windows
//   of the groups of one wavefront for one round lie side by side
//   (wave_off[w] + round) * tpw * 16 elements into the arrays, so the whole
//   wavefront stages a round with one contiguous, fully coalesced load per
//   array; wave_off[w + 1] - wave_off[w] is the number of rounds of wave w.
// MARKS = 1 (sliced arrays only): every column entry also says how many
//   rows end in front of its nonzero, entry = column | ends << mark_shift, so
//   the kernel never reads row_ptr while it works through a partition: no load
//   of its own sits between the window prefetch and the gathers.
// MARKS = 2: entry = column | streamed << mark_shift | ends << (mark_shift + 1);
//   streamed = 1 marks a column outside the set of popular columns whose rows
//   of X are meant to stay in L2: its row is gathered with the streaming hint,
//   so that it does not push a popular row out.
// HOT = true: the column part of an entry is a row slot of the table of X rows
//   that the workgroup keeps in LDS (see below).
// PATTERN = 1: every nonzero counts 1 (val is not read): rows of X are added
//   up.  PATTERN = 2: also, a finished row r is multiplied by row_scale[r]
//   where it is written to Y (the carry records stay unscaled, the fix-up
//   kernel scales).  Plans with degree weights use them: X arrives scaled by
//   the column factor; the row factor is row_scale (2, untiled plans) or is
//   applied when the partial rows are summed (1, tiled plans).
template <typename T, typename TOut, int VEC, bool POW2, int BATCH, bool SLICED, bool HOT, int MARKS, int RPL, int PATTERN = 0>
__global__ __launch_bounds__(64 * (HOT ? kHotWavesPerBlock : kWavesPerBlock)) void mp_spmm_kernel(
    const int *__restrict__ row_ptr, const int *__restrict__ col_idx, const T *__restrict__ val,
    const T *__restrict__ X, TOut *__restrict__ Y, const int *__restrict__ coord_x,
    const int *__restrict__ coord_y, const int *__restrict__ wave_off, int nnz, int K, int P,
    int lanes_log2, int tpw, int wave_begin, int wave_end, int row_shift, int *__restrict__ ws_head_row,
    float *__restrict__ ws_head, float *__restrict__ ws_tail, const int *__restrict__ hot_cols,
    const int *__restrict__ seg_part_off, int num_hot_segs, int hot_rows, const int *__restrict__ hot_block_wave,
    int hot_blocks, int mark_shift, const float *__restrict__ row_scale)
{
    static_assert(!MARKS || SLICED, "row marks live in the sliced arrays");
    static_assert(!PATTERN || MARKS, "pattern mode is built for plans with row marks");
    static_assert(!HOT || MARKS, "the hot launch reads marked entries");
    static_assert(MARKS != 2 || POW2, "streamed entries need the 32-bit offsets of a power-of-two pitch");
    constexpr int WPB = HOT ? kHotWavesPerBlock : kWavesPerBlock;
    using XO = XOps<T, VEC>;
    using Raw = typename XO::Raw;
    constexpr int kCombine = 64 * VEC;  // floats per wave for the head partials (and for the tails)
    constexpr int kStage = (kCombine > 2 * 16 * kWindow) ? kCombine : 2 * 16 * kWindow;
    __shared__ float s_stage[WPB][kStage];   // windows; at the end, the tail partials
    __shared__ float s_heads[WPB][kCombine]; // first finished row of every group
    __shared__ int s_hrow[WPB][16];
    extern __shared__ __align__(16) char s_hot[];  // HOT: the hot rows of X of this block's column slab

    const int wib = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    // Workgroups are dealt round-robin to the 8 XCDs.  Give XCD k the k-th
    // contiguous eighth of the partitions, so that the wavefronts sharing an L2
    // work on neighbouring rows (and, in a tiled plan, on the same column slab).
    const int blocks_per_xcd = gridDim.x / kXcds;
    const int lblock = (blockIdx.x % kXcds) * blocks_per_xcd + blockIdx.x / kXcds;
    int w = wave_begin + lblock * WPB + wib;
    int w_stop = wave_end;
    if constexpr (HOT) {
        // A hot block works through the wavefront-sized pieces [hot_block_wave[b],
        // hot_block_wave[b + 1]) of one hot segment, 16 at a time: it copies that
        // slab's hot rows of X into LDS once; the sliced column array then holds
        // LDS row slots instead of column ids.
        if (lblock >= hot_blocks) return;  // whole block
        const int w0 = hot_block_wave[lblock];
        w_stop = hot_block_wave[lblock + 1];
        if (w0 >= w_stop) return;  // whole block
        w = w0 + wib;
        const int p0 = w0 * tpw;
        int lo = 0, hi = num_hot_segs - 1;
        while (lo < hi) {  // largest hot segment g with seg_part_off[g] <= p0
            int mid = (lo + hi + 1) >> 1;
            if (seg_part_off[mid] <= p0) lo = mid; else hi = mid - 1;
        }
        const int *cols = hot_cols + (size_t)lo * hot_rows;
        const int vec_per_row = (int)(((size_t)K * sizeof(T)) >> 4);
        const int total = hot_rows * vec_per_row;
        const float4 *xsrc = reinterpret_cast<const float4 *>(X);
        float4 *dst = reinterpret_cast<float4 *>(s_hot);
        for (int i = threadIdx.x; i < total; i += 64 * WPB) {
            const int r = i / vec_per_row;
            const int c = cols[r];
            if (c >= 0) dst[i] = xsrc[(size_t)c * vec_per_row + (i - r * vec_per_row)];
        }
        __syncthreads();
    }
    if (w >= w_stop) return;

    const int L = 1 << lanes_log2;
    const int g = lane >> lanes_log2;
    const int s = lane & (L - 1);
    const int KT = L * VEC;  // columns covered by one pass of the wave
    const int kcol = blockIdx.y * KT + s * VEC;
    const bool col_ok = kcol < K;
    // lanes beyond K gather column 0 (a valid address) and never store
    const Gather<T, VEC, POW2> gx{reinterpret_cast<const char *>(X), (size_t)K * sizeof(T),
                                  col_ok ? (unsigned)(kcol * sizeof(T)) : 0u, row_shift};

    // all of X below 4 GiB (what POW2 promises), 32-bit elements, no swizzle
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(X), 0, 0xffffffff, 0x00020000);
    // the row of X that a column entry names
    auto gather = [&](int entry, unsigned mask, int shift) -> Raw {
        const int c = MARKS ? (int)((unsigned)entry & mask) : entry;
        if constexpr (HOT) {
            return *reinterpret_cast<const Raw *>(s_hot + (((unsigned)c << row_shift) | gx.col_byte));
        } else if constexpr (MARKS == 2) {
            return gx.load_hinted(x_rsrc, c, (((unsigned)entry >> shift) & 1u) != 0);
        } else {
            return gx.load(c);
        }
    };

    int *s_col_wave = reinterpret_cast<int *>(&s_stage[wib][0]);
    float *s_val_wave = &s_stage[wib][16 * kWindow];
    const int *s_col = s_col_wave + g * kWindow;
    const float *s_val = s_val_wave + g * kWindow;
    float *my_head = &s_heads[wib][g * KT + s * VEC];

    for (;;) {  // one pass per wavefront-sized piece: one for a cold block, many for a hot one
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
    // The row end after it is loaded ahead, so that finishing a row does not
    // wait on memory.
    auto row_end_at = [&](int xx) { return (!MARKS && xx < x_end) ? row_ptr[xx] : INT_MAX; };
    [[maybe_unused]] int row_end = row_end_at(x), row_end1 = row_end_at(x + 1);
    [[maybe_unused]] const unsigned mark_mask = (1u << mark_shift) - 1u;

    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    int head_row = -1;
    [[maybe_unused]] float cur_scale = 1.f;  // PATTERN = 2: row_scale of the row in progress
    if constexpr (PATTERN == 2) {
        if (part_ok && x - 1 < x_end) cur_scale = row_scale[x - 1];
    }

    auto emit = [&]() {
        const int row = x - 1;
        if (head_row < 0) {
            head_row = row;
#pragma unroll
            for (int i = 0; i < VEC; ++i) my_head[i] = acc[i];
        } else if (col_ok) {
            if constexpr (PATTERN == 2) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[i] *= cur_scale;
            }
            store_acc<VEC, !HOT>(Y + (size_t)row * K + kcol, acc);
        }
        if constexpr (PATTERN == 2) {
            // the factor of the row that starts now, requested a whole row ahead of its use
            if (x < x_end) cur_scale = row_scale[x];
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        ++x;
        if constexpr (!MARKS) {
            row_end = row_end1;
            row_end1 = row_end_at(x + 1);
        }
    };
    // rows that end in front of nonzero idx (entry: what the column array holds for it)
    auto finish_rows = [&](int idx, int entry) {
        if constexpr (MARKS) {
            for (unsigned e = (unsigned)entry >> (mark_shift + (MARKS == 2 ? 1 : 0)); e != 0; --e) emit();
        } else {
            while (idx == row_end) emit();
        }
    };

    int wbase = y_begin;
    // sliced staging: lane l moves elements [4l, 4l + 4) of the wave's round block
    const int round_elems = tpw * kWindow;
    const bool stager = SLICED ? (4 * lane < round_elems) : (s < 4);

    // one staged window of every group: gather, finish rows, accumulate
    auto consume = [&](int nvalid) {
        if (__all(nvalid == kWindow)) {
            // every group of the wave has a full window: no bounds to test
#pragma unroll
            for (int b = 0; b < kWindow; b += BATCH) {
                Raw xr[BATCH];
                int ent[BATCH];
                float av[BATCH];
#pragma unroll
                for (int j = 0; j < BATCH; ++j) {
                    ent[j] = s_col[b + j];
                    av[j] = PATTERN ? 1.0f : s_val[b + j];
                    xr[j] = gather(ent[j], mark_mask, mark_shift);
                }
#pragma unroll
                for (int j = 0; j < BATCH; ++j) {
                    finish_rows(wbase + b + j, ent[j]);
                    XO::fma(acc, av[j], xr[j]);
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < kWindow; b += BATCH) {
                Raw xr[BATCH];
                int ent[BATCH];
#pragma unroll
                for (int j = 0; j < BATCH; ++j) {
                    if (b + j < nvalid) {
                        ent[j] = s_col[b + j];
                        xr[j] = gather(ent[j], mark_mask, mark_shift);
                    }
                }
#pragma unroll
                for (int j = 0; j < BATCH; ++j) {
                    if (b + j < nvalid) {
                        finish_rows(wbase + b + j, ent[j]);
                        XO::fma(acc, PATTERN ? 1.0f : s_val[b + j], xr[j]);
                    }
                }
            }
        }
    };

    if constexpr (SLICED) {
        // RPL rounds are loaded at a time, one load ahead: up to 2 * RPL windows of
        // the wavefront are in flight or in registers.  Measured on MI355X, RPL = 1,
        // 2 and 4 run the hot launch (16 wavefronts per CU) at the same speed, so
        // both launches use 1.
        int round = wave_off[w];
        const int round_end = wave_off[w + 1];
        Win nx[RPL];
#pragma unroll
        for (int h = 0; h < RPL; ++h) {
            nx[h].c = make_int4(0, 0, 0, 0);
            nx[h].v = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        auto load_rounds = [&](int r0) {
#pragma unroll
            for (int h = 0; h < RPL; ++h)
                if (stager && r0 + h < round_end) {
                    if constexpr (PATTERN) nx[h].c = load_slice_cols(col_idx, (size_t)(r0 + h) * round_elems + 4 * lane);
                    else nx[h] = load_slice<T>(col_idx, val, (size_t)(r0 + h) * round_elems + 4 * lane);
                }
        };
        load_rounds(round);
        while (round < round_end) {
            Win cu[RPL];
#pragma unroll
            for (int h = 0; h < RPL; ++h) cu[h] = nx[h];
            load_rounds(round + RPL);
#pragma nounroll
            for (int h = 0; h < RPL && round < round_end; ++h) {
                const int nvalid = min(kWindow, y_end - wbase);  // <= 0 for a group that is done
                if (stager) {
                    *reinterpret_cast<int4 *>(s_col_wave + 4 * lane) = cu[0].c;
                    if constexpr (!PATTERN) *reinterpret_cast<float4 *>(s_val_wave + 4 * lane) = cu[0].v;
                }
                wave_lds_sync();
                consume(nvalid);
                wbase += kWindow;
                ++round;
#pragma unroll
                for (int q = 0; q + 1 < RPL; ++q) cu[q] = cu[q + 1];
                wave_lds_sync();
            }
        }
    } else {
        Win pw;
        pw.c = make_int4(0, 0, 0, 0);
        pw.v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (stager && wbase < y_end) pw = load_win<T>(col_idx, val, nnz, wbase + 4 * s);
        while (__any(wbase < y_end) != 0) {
            const int nvalid = min(kWindow, y_end - wbase);  // <= 0 for a group that is done
            if (stager && nvalid > 0) {
                *reinterpret_cast<int4 *>(s_col_wave + g * kWindow + 4 * s) = pw.c;
                *reinterpret_cast<float4 *>(s_val_wave + g * kWindow + 4 * s) = pw.v;
            }
            wave_lds_sync();
            // next window: in flight while this one is consumed.  One load site for
            // both paths of consume(): the registers of the window in flight are the
            // same everywhere, and nothing else has to wait for it.
            const int nb = wbase + kWindow;
            if (stager && nb < y_end) pw = load_win<T>(col_idx, val, nnz, nb + 4 * s);
            consume(nvalid);
            wbase += kWindow;
            wave_lds_sync();
        }
    }
    while (x < x_end) emit();  // rows that end exactly where the partition ends

    // ---- combine the groups of this wavefront -------------------------------
    const float *heads = &s_heads[wib][0];
    float *tails = &s_stage[wib][0];
#pragma unroll
    for (int i = 0; i < VEC; ++i) tails[g * KT + s * VEC + i] = acc[i];
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
                    float f = 1.f;
                    if constexpr (PATTERN == 2) f = row_scale[hr];
                    Y[(size_t)hr * K + kc] = (TOut)(v * f);
                }
                carry = t;
            } else {
                carry += t;
            }
        }
        if (first && kc == 0) ws_head_row[w] = -1;
        if (kc_ok) ws_tail[(size_t)w * K + kc] = carry;
    }
    if constexpr (!HOT) {
        break;
    } else {
        w += WPB;
        if (w >= w_stop) break;
        wave_lds_sync();  // the combine above has read what the next piece overwrites
    }
    }
}

// Carry-out fix-up: the first row that ends inside wavefront w also received
// nonzeros from the wavefronts before it, back to (and including) the nearest
// one that itself saw a row end.
template <typename TOut>
__global__ __launch_bounds__(256) void mp_fixup_kernel(const int *__restrict__ ws_head_row,
                                                        const float *__restrict__ ws_head,
                                                        const float *__restrict__ ws_tail,
                                                        TOut *__restrict__ Y, int num_waves, int K,
                                                        const float *__restrict__ row_scale)
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
    if (row_scale) sum *= row_scale[hr];
    Y[(size_t)hr * K + k] = (TOut)sum;
}

// The same fix-up for K a multiple of 4 up to 256, with K / 4 lanes per record
// (16-byte loads) and as many records side by side as fit in a wavefront.  A
// lane walks back over at most kFixupShort records on its own; a row that
// reaches further (a hub row under a small cost spans hundreds of wavefronts)
// is finished by the whole wavefront: it finds the end of the chain 64 records
// per step and adds the tails with all lanes.
constexpr int kFixupShort = 6;

template <typename TOut>
__global__ __launch_bounds__(256) void mp_fixup_wide_kernel(const int *__restrict__ ws_head_row,
                                                             const float *__restrict__ ws_head,
                                                             const float *__restrict__ ws_tail,
                                                             TOut *__restrict__ Y, int num_waves, int K,
                                                             const float *__restrict__ row_scale)
{
    const int lane = threadIdx.x & 63;
    const int lpr = K >> 2;      // lanes per record
    const int slots = 64 / lpr;  // records side by side
    const int slot = lane / lpr, q = lane - slot * lpr;
    const long long first_rec = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * slots;
    if (first_rec >= num_waves) return;  // whole wavefront
    const int w = (int)first_rec + slot;
    const bool valid = slot < slots && w < num_waves;
    const float4 *tail4 = reinterpret_cast<const float4 *>(ws_tail);
    auto add = [](float4 &a, const float4 &b) {
        a.x += b.x;
        a.y += b.y;
        a.z += b.z;
        a.w += b.w;
    };
    // what a row that ends one record back needs, requested at once
    int hr = -1, hprev = 0;
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f), t1 = sum;
    if (valid) {
        hr = ws_head_row[w];
        sum = reinterpret_cast<const float4 *>(ws_head)[(size_t)w * lpr + q];
        if (w > 0) {
            hprev = ws_head_row[w - 1];
            t1 = tail4[(size_t)(w - 1) * lpr + q];
        }
    }
    const bool mine = valid && hr >= 0;
    // chain: records w - 1, w - 2, ... back to and including the nearest one with a row end
    int j = w - 1;
    bool open = mine && j >= 0;
    if (open) {
        add(sum, t1);
        open = hprev < 0;
        --j;
    }
    for (int step = 1; step < kFixupShort; ++step) {
        if (open && j >= 0) {
            const float4 t = tail4[(size_t)j * lpr + q];
            const int hj = ws_head_row[j];
            add(sum, t);
            open = hj < 0;
            --j;
        } else {
            open = false;
        }
    }
    // long chains, one after the other, by the whole wavefront
    unsigned long long todo = __ballot(open && j >= 0 && q == 0);
    while (todo != 0) {
        const int src_lane = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const int jstart = __shfl(j, src_lane, 64);  // next record of that chain
        int len = 0;
        for (int base = jstart; base >= 0; base -= 64) {
            const int jj = base - lane;
            const bool stop = jj < 0 || ws_head_row[jj] >= 0;
            const unsigned long long m = __ballot(stop);
            if (m != 0) {
                const int first = __ffsll((long long)m) - 1;
                len += first + ((base - first) >= 0 ? 1 : 0);
                break;
            }
            len += 64;
        }
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        if (slot < slots) {
            int i = slot;
            for (; i + 3 * slots < len; i += 4 * slots) {
                float4 t[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) t[u] = tail4[(size_t)(jstart - (i + u * slots)) * lpr + q];
#pragma unroll
                for (int u = 0; u < 4; ++u) add(acc, t[u]);
            }
            for (; i < len; i += slots) add(acc, tail4[(size_t)(jstart - i) * lpr + q]);
        }
        float4 total = acc;  // slots added in a fixed order: the result does not depend on timing
        for (int sl = 1; sl < slots; ++sl) {
            const int from = q + sl * lpr;
            float4 v;
            v.x = __shfl(acc.x, from, 64);
            v.y = __shfl(acc.y, from, 64);
            v.z = __shfl(acc.z, from, 64);
            v.w = __shfl(acc.w, from, 64);
            add(total, v);
        }
        float4 v;  // from the lanes of slot 0 to the lanes that own the row
        v.x = __shfl(total.x, q, 64);
        v.y = __shfl(total.y, q, 64);
        v.z = __shfl(total.z, q, 64);
        v.w = __shfl(total.w, q, 64);
        if (slot * lpr == src_lane && slot < slots) add(sum, v);
    }
    if (mine) {
        if (row_scale) {
            const float f = row_scale[hr];
            sum.x *= f;
            sum.y *= f;
            sum.z *= f;
            sum.w *= f;
        }
        TOut *out = Y + (size_t)hr * K + 4 * q;
        out[0] = (TOut)sum.x;
        out[1] = (TOut)sum.y;
        out[2] = (TOut)sum.z;
        out[3] = (TOut)sum.w;
    }
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
inline int scan_exclusive_inplace(int *data, int n, int *sums, hipStream_t st)
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
// Launch helpers shared by the entry points
// ---------------------------------------------------------------------------
inline bool aligned_to(const void *p, unsigned a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// log2 of the row pitch in bytes when the fast addressing applies, else -1.
inline int pow2_row_shift(int n_rows, int K, int elem_bytes)
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

inline int make_spmm_shape(int n_rows, int K, int P, int tpw, int elem_bytes, SpmmShape &sh)
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

inline size_t carry_bytes_for(int num_waves, int K)
{
    size_t rows = ((size_t)num_waves + 63) / 64 * 64;
    return rows * sizeof(int) + 2 * (size_t)num_waves * K * sizeof(float);
}

// Gathers in flight per lane between waits: 4 (fewer registers mean more resident wavefronts,
// which is what keeps the L1's request queue full; 2 and 8 measured the same or worse on MI355X).
constexpr int kGatherBatch = 4;

// What a plan adds to a launch: sliced arrays, and optionally the hot launch.
struct PlanLaunch {
    const int *wave_off = nullptr;      // nullptr: CSR arrays
    int hot_waves = 0;                  // waves [0, hot_waves) gather from LDS
    int hot_rows = 0;                   // rows of X per hot table
    const int *hot_cols = nullptr;      // [hot segments][hot_rows] column ids, -1 = unused slot
    const int *seg_part_off = nullptr;  // first partition of every hot segment
    int num_hot_segs = 0;
    const int *hot_block_wave = nullptr;  // [hot_blocks + 1] wave range of every hot workgroup
    int hot_blocks = 0;
    size_t hot_lds_bytes = 0;
    int mark_shift = 0;      // > 0: entries of the (cold) sliced column array carry row marks above this bit
    int hot_mark_shift = 0;  // the same for the hot waves
    bool pattern = false;             // every nonzero counts 1, val is not read (plans with degree weights)
    const float *row_scale = nullptr; // pattern: factor of every finished row (nullptr: none, e.g. partial rows of a tiled plan)
    bool streamed_flag = false;  // the bit at mark_shift says "gather with the streaming hint", row marks sit one bit higher
};

template <typename T, typename TOut, int VEC>
int launch_spmm(const int *row_ptr, const int *col_idx, const T *val, const T *X, TOut *Y, int nnz, int K, int P,
                const int *cx, const int *cy, const PlanLaunch &pl, const SpmmShape &sh, void *ws, unsigned phases,
                hipStream_t st)
{
    const int W = sh.num_waves;
    size_t rows = ((size_t)W + 63) / 64 * 64;
    int *ws_head_row = static_cast<int *>(ws);
    float *ws_head = reinterpret_cast<float *>(ws_head_row + rows);
    float *ws_tail = ws_head + (size_t)W * K;
    const int *wave_off = pl.wave_off;
    if (pl.pattern && (sizeof(T) != 4 || !wave_off || pl.mark_shift <= 0)) return MPS_ERR_UNSUPPORTED;
    if (phases & MPS_PHASE_MAIN) {
#define MPS_LAUNCH_MAIN(POW2, BATCH, SLICED, HOT, MARKS, WB, WE, WPB, LDS, SHIFT)  /* MARKS: 0, 1 or 2 */                                \
    do {                                                                                                          \
        const int nblocks_ = (HOT) ? pl.hot_blocks : ((WE) - (WB) + (WPB)-1) / (WPB);                             \
        dim3 grid_((nblocks_ + kXcds - 1) / kXcds * kXcds, sh.ls.col_tiles);                                      \
        if constexpr ((MARKS) != 0 && sizeof(T) == 4) {                                                           \
            if (pl.pattern && pl.row_scale) {                                                                     \
                hipLaunchKernelGGL((mp_spmm_kernel<T, TOut, VEC, POW2, BATCH, SLICED, HOT, MARKS,                 \
                                                   (HOT) ? kHotRoundsPerLoad : 1, 2>), grid_,                     \
                                   dim3(64 * (WPB)), LDS, st, row_ptr, col_idx, val, X, Y, cx, cy, wave_off, nnz, \
                                   K, P, sh.ls.lanes_log2, sh.tpw, WB, WE, sh.row_shift, ws_head_row, ws_head,    \
                                   ws_tail, pl.hot_cols, pl.seg_part_off, pl.num_hot_segs, pl.hot_rows,           \
                                   pl.hot_block_wave, pl.hot_blocks, SHIFT, pl.row_scale);                        \
                break;                                                                                            \
            }                                                                                                     \
            if (pl.pattern) {                                                                                     \
                hipLaunchKernelGGL((mp_spmm_kernel<T, TOut, VEC, POW2, BATCH, SLICED, HOT, MARKS,                 \
                                                   (HOT) ? kHotRoundsPerLoad : 1, 1>), grid_,                     \
                                   dim3(64 * (WPB)), LDS, st, row_ptr, col_idx, val, X, Y, cx, cy, wave_off, nnz, \
                                   K, P, sh.ls.lanes_log2, sh.tpw, WB, WE, sh.row_shift, ws_head_row, ws_head,    \
                                   ws_tail, pl.hot_cols, pl.seg_part_off, pl.num_hot_segs, pl.hot_rows,           \
                                   pl.hot_block_wave, pl.hot_blocks, SHIFT, nullptr);                             \
                break;                                                                                            \
            }                                                                                                     \
        }                                                                                                         \
        hipLaunchKernelGGL((mp_spmm_kernel<T, TOut, VEC, POW2, BATCH, SLICED, HOT, MARKS, (HOT) ? kHotRoundsPerLoad : 1>), grid_, \
                           dim3(64 * (WPB)), LDS, st, row_ptr, col_idx, val, X, Y, cx, cy, wave_off, nnz, K, P,   \
                           sh.ls.lanes_log2, sh.tpw, WB, WE, sh.row_shift, ws_head_row, ws_head, ws_tail,         \
                           pl.hot_cols, pl.seg_part_off, pl.num_hot_segs, pl.hot_rows, pl.hot_block_wave,         \
                           pl.hot_blocks, SHIFT, nullptr);                                                        \
    } while (0)
        if (pl.hot_waves > 0) {
            // hot launch: only built for power-of-two pitches and vector lanes (VEC > 1)
            if constexpr (VEC > 1) {
                if (pl.hot_mark_shift <= 0) return MPS_ERR_INVALID_ARG;
                // (the kernel's dynamic LDS limit was raised when the plan was made: allow_hot_lds)
                MPS_LAUNCH_MAIN(true, kGatherBatch, true, true, 1, 0, pl.hot_waves, kHotWavesPerBlock, pl.hot_lds_bytes,
                                pl.hot_mark_shift);
            } else {
                return MPS_ERR_UNSUPPORTED;
            }
        }
        const int cold_begin = pl.hot_waves;
        if (cold_begin < W) {
            if (wave_off && pl.mark_shift > 0 && pl.streamed_flag) {
                if (sh.row_shift < 0) return MPS_ERR_INVALID_ARG;  // plans set the flag for power-of-two pitches only
                MPS_LAUNCH_MAIN(true, kGatherBatch, true, false, 2, cold_begin, W, kWavesPerBlock, 0, pl.mark_shift);
            } else if (wave_off && pl.mark_shift > 0) {
                if (sh.row_shift >= 0) MPS_LAUNCH_MAIN(true, kGatherBatch, true, false, 1, cold_begin, W, kWavesPerBlock, 0, pl.mark_shift);
                else MPS_LAUNCH_MAIN(false, kGatherBatch, true, false, 1, cold_begin, W, kWavesPerBlock, 0, pl.mark_shift);
            } else if (wave_off) {
                if (sh.row_shift >= 0) MPS_LAUNCH_MAIN(true, kGatherBatch, true, false, 0, cold_begin, W, kWavesPerBlock, 0, 0);
                else MPS_LAUNCH_MAIN(false, kGatherBatch, true, false, 0, cold_begin, W, kWavesPerBlock, 0, 0);
            } else {
                if (sh.row_shift >= 0) MPS_LAUNCH_MAIN(true, kGatherBatch, false, false, 0, 0, W, kWavesPerBlock, 0, 0);
                else MPS_LAUNCH_MAIN(false, kGatherBatch, false, false, 0, 0, W, kWavesPerBlock, 0, 0);
            }
        }
#undef MPS_LAUNCH_MAIN
        MPS_HIP_TRY(hipGetLastError());
    }
    if (phases & MPS_PHASE_FIXUP) {
        if (K % 4 == 0 && K <= 256) {
            const int per_wave = 64 / (K / 4);  // records per wavefront
            const long long fix_waves = ((long long)W + per_wave - 1) / per_wave;
            hipLaunchKernelGGL((mp_fixup_wide_kernel<TOut>), dim3((unsigned)((fix_waves + 3) / 4)), dim3(256), 0, st,
                               ws_head_row, ws_head, ws_tail, Y, W, K, pl.row_scale);
        } else {
            long long threads = (long long)W * K;
            unsigned blocks = (unsigned)((threads + 255) / 256);
            hipLaunchKernelGGL((mp_fixup_kernel<TOut>), dim3(blocks), dim3(256), 0, st, ws_head_row, ws_head, ws_tail,
                               Y, W, K, pl.row_scale);
        }
        MPS_HIP_TRY(hipGetLastError());
    }
    return MPS_OK;
}

// Raises the dynamic LDS limit of the hot instantiation that launch_spmm<T, TOut, VEC> uses; called once
// per plan, so that a product launches kernels only (it may run under stream capture).  The limit is one
// value per kernel: it is set to what a CU holds, whatever this plan needs, so that a plan with a smaller
// table cannot lower it under an earlier plan that is still in use.
constexpr size_t kHotLdsLimit = 160 * 1024;
inline int raise_dynamic_lds_limit(const void *kernel, size_t bytes)
{
    hipFuncAttributes attr;
    MPS_HIP_TRY(hipFuncGetAttributes(&attr, kernel));
    if (attr.sharedSizeBytes + bytes > kHotLdsLimit) return MPS_ERR_UNSUPPORTED;
    // all that a CU holds beside the kernel's own static buffers
    MPS_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kHotLdsLimit - attr.sharedSizeBytes)));
    return MPS_OK;
}
template <typename T, typename TOut, int VEC>
int allow_hot_lds_for(size_t bytes)
{
    if constexpr (VEC > 1) {
        auto kern = mp_spmm_kernel<T, TOut, VEC, true, kGatherBatch, true, true, 1, kHotRoundsPerLoad>;
        int rc = raise_dynamic_lds_limit(reinterpret_cast<const void *>(kern), bytes);
        if (rc != MPS_OK) return rc;
        if constexpr (sizeof(T) == 4) {
            // hot columns come with tiled plans, whose partial rows are scaled when they are summed
            auto pattern_kern = mp_spmm_kernel<T, TOut, VEC, true, kGatherBatch, true, true, 1, kHotRoundsPerLoad, 1>;
            rc = raise_dynamic_lds_limit(reinterpret_cast<const void *>(pattern_kern), bytes);
            if (rc != MPS_OK) return rc;
        }
        return MPS_OK;
    } else {
        return MPS_ERR_UNSUPPORTED;
    }
}

template <typename T, typename TOut>
int allow_hot_lds(const SpmmShape &sh, size_t bytes)
{
    if (sh.ls.vec == 1) return allow_hot_lds_for<T, TOut, 1>(bytes);
    if constexpr (sizeof(T) == 2) {
        if (sh.ls.vec == 4) return allow_hot_lds_for<T, TOut, 4>(bytes);
    }
    return allow_hot_lds_for<T, TOut, 16 / (int)sizeof(T)>(bytes);
}

template <typename T, typename TOut>
int launch_spmm_any(const int *row_ptr, const int *col_idx, const T *val, const T *X, TOut *Y, int nnz, int K,
                    int P, const int *cx, const int *cy, const PlanLaunch &pl, const SpmmShape &sh, void *ws,
                    unsigned phases, hipStream_t st)
{
    if (sh.ls.vec == 1)
        return launch_spmm<T, TOut, 1>(row_ptr, col_idx, val, X, Y, nnz, K, P, cx, cy, pl, sh, ws, phases, st);
    if constexpr (sizeof(T) == 2) {
        if (sh.ls.vec == 4)  // narrow fp16 rows: 8 bytes per lane
            return launch_spmm<T, TOut, 4>(row_ptr, col_idx, val, X, Y, nnz, K, P, cx, cy, pl, sh, ws, phases, st);
    }
    return launch_spmm<T, TOut, 16 / (int)sizeof(T)>(row_ptr, col_idx, val, X, Y, nnz, K, P, cx, cy, pl, sh, ws,
                                                     phases, st);
}

}  // namespace

#endif
