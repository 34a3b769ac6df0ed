// Sweep plans, device side: the kernel that walks the layout of
// mpspmm_sweep.hpp, the fix-up of rows that were cut across panels, and the
// plan object's device arrays.
//
// Same arithmetic as the reference kernel (src/MergePathSpMM.cu:426-477: one
// fp32 accumulator per output column, a product added per nonzero; the fp16
// variant src/MergePathSpMM_fp16.cu:427-477 with fp32 sums, as the oracle's
// orc_spmm_f64_f16in prescribes), with explicit values in place of the degree
// product (:450, :459-460).  What differs is the order of the nonzeros (by
// column within a wavefront, so that the gathers of the whole chip stay within
// a narrow range of X) and where a row is summed (an LDS accumulator row that
// one wavefront owns, instead of atomics on Y, :445, :477).
#include "mpspmm_device.hpp"
#include "mpspmm_sweep.hpp"

#include <new>

namespace mps_sw {

struct DevicePlan {
    Layout host;  // the small tables stay filled; stream and src are released after the upload
    uint32_t *stream = nullptr;
    int *src = nullptr;
    int *panel_ptr = nullptr, *rows = nullptr, *piece_ptr = nullptr, *wave_meta = nullptr, *panel_rounds = nullptr;
    int *split_row = nullptr, *split_ptr = nullptr;
    float *partial = nullptr;  // [partial rows][K] fp32 sums of the sub-rows of split rows
    size_t lds_bytes = 0, device_bytes = 0, slots = 0;
    int round_panels = 256;  // panels are made in multiples of this: one round of workgroups
    bool built_on_device = false;
};

namespace {

typedef unsigned u4_t __attribute__((ext_vector_type(4)));
// An entry stream of at most this size is read with plain loads and stays in the 256 MiB last-level cache from one
// pass over a column tile and from one product to the next; a larger one is read with the streaming hint, which keeps
// it out of there.  Measured on MI355X, R-MAT scale 20, fp32 (a stream of 138 MB), ms per product with the hint /
// with plain loads: K = 16 0.1185 / 0.1052, K = 32 0.1525 / 0.1465, K = 64 0.3125 / 0.3206, K = 128 0.6465 / 0.6130,
// K = 256 1.289 / 1.247; R-MAT scale 22, fp16, K = 64 (563 MB): 0.850 / 0.866.
constexpr size_t kStreamKeepBytes = 160u << 20;
typedef float f4_t __attribute__((ext_vector_type(4)));

// Entry j of the lane-group's window sits in lane j of the quad; all lanes of the quad read it.  (A compiler-made
// DPP move: the compiler keeps the wait states a DPP read needs after a write of its source.)
template <int J>
__device__ __forceinline__ unsigned from_lane(unsigned v)
{
    return (unsigned)__builtin_amdgcn_mov_dpp((int)v, J | (J << 2) | (J << 4) | (J << 6), 0xf, 0xf, true);
}

// 16 bytes of a row of X as fp32 values: 4 floats, or 8 halves widened
template <typename T>
struct Piece;
template <>
struct Piece<float> {
    static constexpr int kVec = 4, kPlanes = 1;
    f4_t raw;
    __device__ __forceinline__ void load(const char *p) { raw = *reinterpret_cast<const f4_t *>(p); }
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned off)
    {
        raw = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
    }
    __device__ __forceinline__ f4_t plane(int) const { return raw; }
};
template <>
struct Piece<half_t> {
    static constexpr int kVec = 8, kPlanes = 2;
    half8_t raw;
    __device__ __forceinline__ void load(const char *p) { raw = *reinterpret_cast<const half8_t *>(p); }
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, unsigned off)
    {
        raw = __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
    }
    __device__ __forceinline__ f4_t plane(int q) const
    {
        return q == 0 ? f4_t{(float)raw[0], (float)raw[1], (float)raw[2], (float)raw[3]}
                      : f4_t{(float)raw[4], (float)raw[5], (float)raw[6], (float)raw[7]};
    }
};

// A lane's 16 bytes of a row of Y (or of a partial row): `valid` of the kVec sums, the others lie past the row's end.
// Rows whose pitch is no multiple of 16 bytes start anywhere on a dword boundary.
template <typename TOut, int VEC>
__device__ __forceinline__ void store_piece(TOut *p, const float (&sum)[VEC], int valid)
{
    if (valid >= VEC) {
        store_acc<VEC, true>(p, sum);
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e)
            if (e < valid) __builtin_nontemporal_store((TOut)sum[e], p + e);
    }
}

// T: element type of X and Y.  L: lanes per lane-group (16 L bytes of a row of X per tile).  FAR: X is addressed with
// 64-bit pointers; otherwise (X below 4 GiB, fewer than 2^24 rows) with a 32-bit offset that one 24-bit
// multiply-add forms, through a buffer descriptor that knows the size of X.
// K is any number of elements that fills whole dwords: a row of X is ceil(16 L-byte tiles), and in the last tile
//   * a lane whose 16 bytes begin past the row's end reads the tile's first 16 bytes instead (the line that lane 0
//     of its lane-group asks for anyway) and adds them to a part of the accumulator row that is never written out;
//   * a lane whose 16 bytes begin inside the row and end past it reads the first elements of the next row with its
//     own last ones and never writes those sums out either.  Past the last row of X there is no next row: the buffer
//     descriptor's range check, which works dword by dword on such loads, returns zeros there and requests nothing.
//     (With 64-bit pointers nothing checks the range: FAR plans are built for rows of whole 16 bytes only.)
// LDS: kPlanes planes of (acc_rows + 1) x L float4: plane q holds elements 4 q .. 4 q + 3 of every lane's 16 bytes, so
// that one 16-byte LDS access per lane covers a plane's row exactly like an fp32 row.
template <typename T, int L, int TOGETHER, bool FAR>
__global__ __launch_bounds__(kThreads) void sw_spmm_kernel(const uint4 *__restrict__ stream, const int2 *__restrict__ wave_meta,
                                                            const int *__restrict__ panel_rounds,
                                                            const int *__restrict__ panel_ptr, const int *__restrict__ rows,
                                                            const int *__restrict__ piece_ptr, const T *__restrict__ X,
                                                            T *__restrict__ Y, float *__restrict__ partial, int n, int K,
                                                            int acc_rows, int col_bits, int bank_rows, int stream_keep, int tiles, int round_panels)
{
    extern __shared__ __align__(16) char smem[];
    f4_t *acc4 = reinterpret_cast<f4_t *>(smem);
    using P = Piece<T>;
    constexpr int GPW = 64 / L;        // lane-groups of a wavefront
    constexpr int RQ = GPW * kWin;     // 16-byte units of a round
    // a workgroup barrier every so many rounds (see below): 1 for 64-byte rows, 2 for 128-byte tiles of fp32, 4 of fp16
    constexpr int kSync = L == 4 ? 1 : sizeof(T) == 4 ? 2 : kSyncRounds;
    constexpr bool kPairPrio = L == 8 && sizeof(T) == 2;  // the wavefronts' priorities move on with every entry of a round
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroups in the order of a one-dimensional grid: a round of panels at its first column tile, the same
    // panels at the next tile, ... then the next round of panels - what a round of panels read of the entry stream
    // is read again at once for the next tile.  (Tile by tile over all panels instead, as a two-dimensional grid
    // orders them: R-MAT scale 20, fp32, K = 64 / 128 / 256 2.8 / 4.0 / 3.7 % slower.)
    // (Kernels for 64-byte tiles keep the two-dimensional grid: their plans of one tile lose 2-4 % by the arithmetic.)
    int b = blockIdx.x, tile = 0;
    if constexpr (L == 4) {
        tile = blockIdx.y;
        tiles = gridDim.y;
    } else if (tiles > 1) {
        const int span = round_panels * tiles, grp = (int)blockIdx.x / span, within = (int)blockIdx.x - grp * span;
        tile = within / round_panels;
        b = grp * round_panels + (within - tile * round_panels);
    }
    const int g = lane / L, c = lane % L, s = lane & 3;
    const int plane_stride = (acc_rows + 1) * L;  // float4 units
    const f4_t zero = {0.f, 0.f, 0.f, 0.f};
    for (int i = tid; i < plane_stride * P::kPlanes; i += kThreads) acc4[i] = zero;

    const int2 wm = wave_meta[b * kWaves + wave];
    const int rounds = __builtin_amdgcn_readfirstlane(wm.y);
    const int most = panel_rounds[b];
    const unsigned cmask = (1u << col_bits) - 1u;
    // this lane's 16 bytes of a row of X: row pitch K elements, tile `tile`, piece c
    const unsigned row_pitch = (unsigned)K * (unsigned)sizeof(T);
    const unsigned lane_off = (unsigned)c * 16u, tile_off = (unsigned)tile * (16u * L);
    const unsigned x_off = tile_off + lane_off < row_pitch ? tile_off + lane_off : tile_off;
    [[maybe_unused]] const char *xb = reinterpret_cast<const char *>(X) + x_off;
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(X), 0, FAR ? 0xffffffffu : (unsigned)n * row_pitch, 0x00020000);
    const unsigned plane_bytes = (unsigned)plane_stride * 16u;

    // The entries are read once per pass over a column tile, through a buffer descriptor (the base of the wavefront's
    // run in scalar registers, the cache policy as an operand of the load).  stream_keep: with plain loads, so that a
    // stream that fits stays in the 256 MiB last-level cache from one tile's pass and one product to the next;
    // otherwise with the streaming hint, which keeps it out of there.
    const __amdgpu_buffer_rsrc_t s_rsrc = [&]() {
        const unsigned long long a = (unsigned long long)(stream + (size_t)wm.x * RQ);  // the same in all lanes
        const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
        return __builtin_amdgcn_make_buffer_rsrc((void *)(((unsigned long long)hi << 32) | lo), 0, 0xffffffff, 0x00020000);
    }();
    const unsigned s_off = (unsigned)(g * kWin + s) * 16u;
    auto stream_load = [&](int r) {
        const int off = (int)(s_off + (unsigned)r * (RQ * 16u));
        const u4_t t = stream_keep ? __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, off, 0, 0)
                                   : __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, off, 0, 2);
        return make_uint4(t[0], t[1], t[2], t[3]);
    };
    // The row of X of entry k of a round (of 8 entries per lane-group), and where in the LDS (plane 0) this lane adds it.
    P x[kRoundInstr];
    unsigned at[kRoundInstr];
#define SW_GATHER(k, WORD, j, CM)                                                             \
    {                                                                                        \
        const unsigned w = from_lane<j>(WORD);                                               \
        at[k] = (w >> col_bits) * (16u * L) + lane_off;                                      \
        if constexpr (FAR) {                                                                 \
            x[k].load(xb + (size_t)(w & (CM)) * row_pitch);                                  \
        } else {                                                                             \
            x[k].load(x_rsrc, __umul24(w & (CM), row_pitch) + x_off);                        \
        }                                                                                    \
    }
    // One entry after the other: read the accumulator row, add, write it back.  The LDS serves a wavefront's
    // accesses in order, so an entry sees what the entry before it wrote; the lane-groups of one instruction hold
    // different rows (the builder's rule); no other wavefront touches this one's rows.  TOGETHER == 2: entry q of
    // window A and entry q of window B at the same time (the builder keeps their rows apart too), which halves
    // the chain of LDS round trips.
#define SW_FMA(a, v, xv)            \
    a[0] = fmaf(v, xv[0], a[0]);    \
    a[1] = fmaf(v, xv[1], a[1]);    \
    a[2] = fmaf(v, xv[2], a[2]);    \
    a[3] = fmaf(v, xv[3], a[3]);
#define SW_AT(k, q) reinterpret_cast<f4_t *>(smem + at[k] + (q) * plane_bytes)
#define SW_ADD(k, VAL, j)                                                              \
    {                                                                                  \
        const float v = __uint_as_float(from_lane<j>(VAL));                            \
        _Pragma("unroll") for (int q = 0; q < P::kPlanes; ++q)                         \
        {                                                                              \
            const f4_t xv = x[k].plane(q);                                             \
            f4_t a = *SW_AT(k, q);                                                     \
            SW_FMA(a, v, xv)                                                           \
            *SW_AT(k, q) = a;                                                          \
        }                                                                              \
    }
#define SW_ADD2(j)                                                                     \
    {                                                                                  \
        const float va = __uint_as_float(from_lane<j>(cu.y)), vb = __uint_as_float(from_lane<j>(cu.w)); \
        f4_t a[P::kPlanes], b[P::kPlanes];                                             \
        _Pragma("unroll") for (int q = 0; q < P::kPlanes; ++q)                         \
        {                                                                              \
            a[q] = *SW_AT(j, q);                                                       \
            b[q] = *SW_AT(kWin + j, q);                                                \
        }                                                                              \
        _Pragma("unroll") for (int q = 0; q < P::kPlanes; ++q)                         \
        {                                                                              \
            const f4_t xa = x[j].plane(q), xw = x[kWin + j].plane(q);                  \
            SW_FMA(a[q], va, xa)                                                       \
            SW_FMA(b[q], vb, xw)                                                       \
            *SW_AT(j, q) = a[q];                                                       \
            *SW_AT(kWin + j, q) = b[q];                                                \
        }                                                                              \
    }
    // Entry k of round r is added up, and the registers that held its row of X at once take the request for entry k
    // of round r + 1: every row of X is asked for a round ahead of its use, in one set of registers, and the entries
    // of round r + 2 are read meanwhile.  No branch goes around a load (where two paths with different loads in
    // flight meet, the compiler waits for all of them): past the wavefront's last round the loop reads that round's
    // entries a second time, asks for row 0 of X in place of their rows, and drops both.
    if (rounds > 0) {
        const int last = rounds - 1;
        uint4 cu = stream_load(0), nx = stream_load(min(1, last));
        SW_GATHER(0, cu.x, 0, cmask) SW_GATHER(1, cu.x, 1, cmask) SW_GATHER(2, cu.x, 2, cmask) SW_GATHER(3, cu.x, 3, cmask)
        SW_GATHER(4, cu.z, 0, cmask) SW_GATHER(5, cu.z, 1, cmask) SW_GATHER(6, cu.z, 2, cmask) SW_GATHER(7, cu.z, 3, cmask)
        for (int r = 0; r < rounds; ++r) {
            // Every few rounds the wavefronts of the workgroup wait for each other (the first time: for the zeroed
            // accumulators): left alone, the oldest wavefront of a SIMD runs ahead of the youngest by a third of the
            // sweep, and the range of X that the chip gathers from at one time no longer fits an L2.
            // (64-byte rows: every round - R-MAT scale 20, fp32, K = 16, a barrier every 1 / 2 / 4 / 8 / 16 / 64 rounds:
            // 0.117 / 0.122 / 0.125 / 0.130 / 0.136 / 0.147 ms per product; 128-byte tiles: every fourth - K = 32
            // 0.162 / 0.161 / 0.158 / 0.166 / 0.173 / 0.190, K = 128 0.672 / 0.671 / 0.658 / 0.681 / 0.700 / 0.758; with
            // the entries of a round in strict order, plain stream loads and the rounds of panels taken through their
            // tiles, every 2 / 4 / 8 rounds: K = 32 0.1343 / 0.1363 / 0.1406, K = 64 0.3020 / 0.3035 / 0.3130, K = 256
            // 1.214 / 1.215 / 1.257 - every second; fp16, K = 64, every 2 / 4 / 8 / 16: 0.863 / 0.852 / 0.862 / 0.866)
            if ((r & (kSync - 1)) == 0) __syncthreads();
            // Between two barriers a SIMD would serve the oldest of its four wavefronts first in every round and the
            // other three would arrive late together.  The priority goes round instead, a round at each rank, the
            // youngest first (launch rank - round).  Measured on MI355X, R-MAT scale 20, fp32, ms per product without
            // / with: K = 16 0.1277 / 0.1257, K = 32 0.1628 / 0.1579, K = 128 0.6857 / 0.6605; R-MAT scale 22, fp16,
            // K = 64 0.916 / 0.915.  (rank + round: 0.126, 0.164, 0.682, 0.912; a step per two or four rounds, or the
            // same rotation begun at another rank: between these and slower than none.)
            // 128-byte tiles: the eight entries of a round are added up and asked for one after the other, in the
            // order written here - the compiler is told not to mix them (fp32: K = 32 0.1563 -> 0.1526, K = 128
            // 0.6577 -> 0.6464 ms per product) -, and for rows of halves the priority moves on a rank with every
            // entry instead of every round (fp16 K = 64: 0.913 -> 0.852; fp32 loses 1 % by that).
#define SW_PRIO(v)                                        \
    switch ((v) & 3) {                                    \
    case 0: __builtin_amdgcn_s_setprio(0); break;         \
    case 1: __builtin_amdgcn_s_setprio(1); break;         \
    case 2: __builtin_amdgcn_s_setprio(2); break;         \
    default: __builtin_amdgcn_s_setprio(3); break;        \
    }
#define SW_NEXT_PAIR(k)                                           \
    if constexpr (kPairPrio) {                                    \
        SW_PRIO(pr - (k))                                         \
    } else if constexpr (L == 8) {                                \
        __builtin_amdgcn_sched_barrier(0);                        \
    }
            const int pr = (wave >> 2) - (kPairPrio ? 8 * r : r);
            SW_PRIO(pr)
            const uint4 cn = nx;
            nx = stream_load(min(r + 2, last));
            const unsigned cm = r < last ? cmask : 0u;  // (past the last round: row 0 of X, eight times)
            if constexpr (TOGETHER == 2) {
                SW_ADD2(0) SW_GATHER(0, cn.x, 0, cm) SW_GATHER(4, cn.z, 0, cm)
                SW_ADD2(1) SW_GATHER(1, cn.x, 1, cm) SW_GATHER(5, cn.z, 1, cm)
                SW_ADD2(2) SW_GATHER(2, cn.x, 2, cm) SW_GATHER(6, cn.z, 2, cm)
                SW_ADD2(3) SW_GATHER(3, cn.x, 3, cm) SW_GATHER(7, cn.z, 3, cm)
            } else {
                SW_ADD(0, cu.y, 0) SW_GATHER(0, cn.x, 0, cm)
                SW_NEXT_PAIR(1)
                SW_ADD(1, cu.y, 1) SW_GATHER(1, cn.x, 1, cm)
                SW_NEXT_PAIR(2)
                SW_ADD(2, cu.y, 2) SW_GATHER(2, cn.x, 2, cm)
                SW_NEXT_PAIR(3)
                SW_ADD(3, cu.y, 3) SW_GATHER(3, cn.x, 3, cm)
                SW_NEXT_PAIR(4)
                SW_ADD(4, cu.w, 0) SW_GATHER(4, cn.z, 0, cm)
                SW_NEXT_PAIR(5)
                SW_ADD(5, cu.w, 1) SW_GATHER(5, cn.z, 1, cm)
                SW_NEXT_PAIR(6)
                SW_ADD(6, cu.w, 2) SW_GATHER(6, cn.z, 2, cm)
                SW_NEXT_PAIR(7)
                SW_ADD(7, cu.w, 3) SW_GATHER(7, cn.z, 3, cm)
            }
            cu = cn;
        }
    }
#undef SW_NEXT_PAIR
#undef SW_PRIO
#undef SW_ADD2
#undef SW_ADD
#undef SW_AT
#undef SW_FMA
#undef SW_GATHER
    // the barriers of the rounds that other wavefronts of the panel still have, and the one before the sums are read
    for (int r = (rounds + kSync - 1) & ~(kSync - 1); r < most; r += kSync) __syncthreads();
    __syncthreads();

    // the panel's rows, once: a row's pieces added up in order, rows without nonzeros as zeros
    const int p0 = panel_ptr[b], nrows = panel_ptr[b + 1] - p0;
    const int *pp = piece_ptr + p0 + b;
    for (int i = tid; i < nrows * L; i += kThreads) {
        const int k = i / L, cc = i % L;
        const int row = rows[p0 + k];
        const int a0 = pp[k], a1 = pp[k + 1];
        float sum[P::kVec];
#pragma unroll
        for (int e = 0; e < P::kVec; ++e) sum[e] = 0.f;
        for (int p = a0; p < a1; ++p) {
            const int vr = p ^ (((p >> 2) ^ (p >> 4) ^ (p >> 6)) & (bank_rows - 1));
#pragma unroll
            for (int q = 0; q < P::kPlanes; ++q) {
                const f4_t a = acc4[q * plane_stride + vr * L + cc];
                sum[4 * q] += a[0];
                sum[4 * q + 1] += a[1];
                sum[4 * q + 2] += a[2];
                sum[4 * q + 3] += a[3];
            }
        }
        const int col0 = tile * (L * P::kVec) + cc * P::kVec;
        if (row < n) {
            if (col0 < K) store_piece<T, P::kVec>(Y + (size_t)row * K + col0, sum, K - col0);
        } else {
            // read again by the fix-up kernel; a partial row has whole tiles
            store_acc<P::kVec, false>(partial + (size_t)(row - n) * ((size_t)tiles * (L * P::kVec)) + col0, sum);
        }
    }
}

// Y[split_row[i]][:] = the sum of its partial rows (pitch Kp floats: whole tiles), in order.
template <typename T>
__global__ __launch_bounds__(256) void sw_fixup_kernel(const int *__restrict__ split_row, const int *__restrict__ split_ptr,
                                                        const float *__restrict__ partial, T *__restrict__ Y, int n_split, int K,
                                                        int Kp)
{
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long long)n_split * K) return;
    const int r = (int)(i / K), e = (int)(i % K);
    float sum = 0.f;
    for (int p = split_ptr[r]; p < split_ptr[r + 1]; ++p) sum += partial[(size_t)p * Kp + e];
    Y[(size_t)split_row[r] * K + e] = (T)sum;
}

// New values into the stream: entry slot i (stream order) holds nonzero src[i].
template <typename T>
__global__ __launch_bounds__(256) void sw_set_values_kernel(const T *__restrict__ val, const int *__restrict__ src, size_t slots,
                                                             uint32_t *__restrict__ stream)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= slots) return;
    const int e = src[i];
    if (e >= 0) stream[2 * i + 1] = __float_as_uint((float)val[e]);
}

__global__ __launch_bounds__(256) void sw_widen_values_kernel(const half_t *__restrict__ in, float *__restrict__ out, size_t n)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (float)in[i];
}

template <typename T, typename A>
int upload(DevicePlan *dp, T **dst, const std::vector<T, A> &src, hipStream_t st)
{
    const size_t bytes = (src.size() ? src.size() : 1) * sizeof(T);
    MPS_HIP_TRY(hipMalloc(reinterpret_cast<void **>(dst), bytes));
    dp->device_bytes += bytes;
    if (!src.empty()) MPS_HIP_TRY(hipMemcpyAsync(*dst, src.data(), src.size() * sizeof(T), hipMemcpyHostToDevice, st));
    return MPS_OK;
}

// 32-bit offsets into X where every row starts below 4 GiB and a column index fits the 24-bit multiply; 64-bit pointers
// otherwise
bool needs_far(const Layout &Lo)
{
    const unsigned long long pitch = (unsigned long long)Lo.K * (unsigned long long)Lo.elem_bytes;
    return Lo.col_bits > 24 || (unsigned long long)Lo.n * pitch > 0xffffff00ull || pitch >= (1ull << 24);
}

// elements of a row in whole tiles: the pitch of the partial rows
int padded_width(const Layout &Lo) { return Lo.tiles * Lo.lanes * (16 / Lo.elem_bytes); }

template <typename T, int L, int TOGETHER, bool FAR>
int launch_main(const DevicePlan *dp, const T *X, T *Y, hipStream_t st)
{
    const Layout &Lo = dp->host;
    // (panels come in whole rounds; a layout that does not keep to that is walked tile by tile, one round of all its panels)
    const int round_panels = dp->round_panels > 0 && Lo.num_panels % dp->round_panels == 0 ? dp->round_panels : Lo.num_panels;
    const dim3 grid = L == 4 ? dim3((unsigned)Lo.num_panels, (unsigned)Lo.tiles) : dim3((unsigned)(Lo.num_panels * Lo.tiles));
    hipLaunchKernelGGL((sw_spmm_kernel<T, L, TOGETHER, FAR>), grid, dim3(kThreads),
                       dp->lds_bytes, st, reinterpret_cast<const uint4 *>(dp->stream),
                       reinterpret_cast<const int2 *>(dp->wave_meta), dp->panel_rounds, dp->panel_ptr, dp->rows, dp->piece_ptr, X,
                       Y, dp->partial, Lo.n, Lo.K, Lo.acc_rows, Lo.col_bits, Lo.bank_rows, dp->slots * 8 <= kStreamKeepBytes ? 1 : 0, Lo.tiles, round_panels);
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

template <typename T, int L, int TOGETHER>
int launch_main(const DevicePlan *dp, const T *X, T *Y, hipStream_t st)
{
    return needs_far(dp->host) ? launch_main<T, L, TOGETHER, true>(dp, X, Y, st) : launch_main<T, L, TOGETHER, false>(dp, X, Y, st);
}

template <typename T>
int spmm_typed(const DevicePlan *dp, const T *X, T *Y, unsigned phases, hipStream_t st)
{
    const Layout &Lo = dp->host;
    if (phases & MPS_PHASE_MAIN) {
        const int rc = Lo.lanes == 8 ? (Lo.together == 2 ? launch_main<T, 8, 2>(dp, X, Y, st) : launch_main<T, 8, 1>(dp, X, Y, st))
                                     : (Lo.together == 2 ? launch_main<T, 4, 2>(dp, X, Y, st) : launch_main<T, 4, 1>(dp, X, Y, st));
        if (rc != MPS_OK) return rc;
    }
    if ((phases & MPS_PHASE_FIXUP) && !Lo.split_row.empty()) {
        const long long threads = (long long)Lo.split_row.size() * Lo.K;
        hipLaunchKernelGGL((sw_fixup_kernel<T>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, dp->split_row,
                           dp->split_ptr, dp->partial, Y, (int)Lo.split_row.size(), Lo.K, padded_width(Lo));
        MPS_HIP_TRY(hipGetLastError());
    }
    return MPS_OK;
}

}  // namespace

void destroy(DevicePlan *dp)
{
    if (!dp) return;
    (void)hipFree(dp->stream);
    (void)hipFree(dp->src);
    (void)hipFree(dp->panel_ptr);
    (void)hipFree(dp->rows);
    (void)hipFree(dp->piece_ptr);
    (void)hipFree(dp->wave_meta);
    (void)hipFree(dp->panel_rounds);
    (void)hipFree(dp->split_row);
    (void)hipFree(dp->split_ptr);
    (void)hipFree(dp->partial);
    delete dp;
}

// Copies the CSR arrays to the host, builds the layout there and uploads it.  The arrays must have passed
// mps_csr_validate.  d_val: fp32 or fp16 by bp.elem_bytes.
int create(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n, int nnz, int K, const BuildParams &bp_in,
           hipStream_t st, DevicePlan **out)
{
    *out = nullptr;
    DevicePlan *dp = new (std::nothrow) DevicePlan;
    if (!dp) return MPS_ERR_UNSUPPORTED;
    int rc = MPS_OK;
    bool on_device = false;
    auto fail = [&](int code) {
        (void)hipStreamSynchronize(st);  // uploads from the layout's host arrays may still be in flight
        destroy(dp);
        return code;
    };
    try {
        BuildParams bp = bp_in;
        if (bp.num_cus <= 0) {
            int dev = 0, cus = 256;
            hipError_t e = hipGetDevice(&dev);
            if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
            bp.num_cus = cus;
        }
        dp->round_panels = bp.num_cus;
        // half values are widened on the device first (exact): both builders take fp32 values
        struct Dev {
            void *p = nullptr;
            ~Dev() { if (p) (void)hipFree(p); }
        } wide;
        hipError_t e = hipSuccess;
        const float *val_src = static_cast<const float *>(d_val);
        if (bp.elem_bytes == 2 && nnz > 0) {
            e = hipMalloc(&wide.p, (size_t)nnz * sizeof(float));
            if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
            hipLaunchKernelGGL(sw_widen_values_kernel, dim3((unsigned)(((size_t)nnz + 255) / 256)), dim3(256), 0, st,
                               static_cast<const half_t *>(d_val), static_cast<float *>(wide.p), (size_t)nnz);
            val_src = static_cast<const float *>(wide.p);
        }
        // panels, listed rows and accumulator rows need row_ptr alone
        std::vector<int> rp((size_t)n + 1);
        e = hipMemcpyAsync(rp.data(), d_row_ptr, ((size_t)n + 1) * sizeof(int), hipMemcpyDeviceToHost, st);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
        if (rp[0] != 0 || rp[(size_t)n] != nnz) return fail(MPS_ERR_INVALID_CSR);
        Bulk<ListedRow> listed_rows;
        rc = plan_panels(rp.data(), n, nnz, K, bp, dp->host, listed_rows);
        if (rc != MPS_OK) return fail(rc);
        // (an X of 4 GiB or more is read through pointers, with nothing to catch the lane that reads past the end of
        // its last row: rows of whole 16 bytes only)
        if (needs_far(dp->host) && ((long long)K * bp.elem_bytes) % 16 != 0) return fail(MPS_ERR_UNSUPPORTED);
        if (!bp.host_build) {
            // the passes over the nonzeros where the nonzeros are
            DeviceStreams ds;
            rc = build_streams_on_device(d_row_ptr, d_col_idx, val_src, bp, dp->host, listed_rows, st, &ds);
            if (rc == MPS_OK) {
                dp->stream = ds.stream;
                dp->src = ds.src;
                dp->slots = ds.slots;
                dp->device_bytes += ds.bytes;
                on_device = true;
            } else {
                (void)hipStreamSynchronize(st);
                (void)hipFree(ds.stream);
                (void)hipFree(ds.src);
                // (the device passes sort two copies of the entries: without room for them, the host's)
                if (rc == MPS_ERR_HIP + (int)hipErrorOutOfMemory) {
                    (void)hipGetLastError();
                    rc = kNeedHost;
                }
                if (rc != kNeedHost) return fail(rc);
            }
        }
        if (!on_device) {
            // the CSR arrays come back into pinned host memory (a pageable target takes ten times as long) and are
            // released as soon as the layout is built
            struct Pinned {
                void *p = nullptr;
                ~Pinned() { if (p) (void)hipHostFree(p); }
            } h_ci, h_val;
            e = hipHostMalloc(&h_ci.p, ((size_t)nnz + 1) * sizeof(int), hipHostMallocDefault);
            if (e == hipSuccess) e = hipHostMalloc(&h_val.p, ((size_t)nnz + 1) * sizeof(float), hipHostMallocDefault);
            if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
            int *ci = static_cast<int *>(h_ci.p);
            float *val = static_cast<float *>(h_val.p);
            if (nnz > 0) e = hipMemcpyAsync(ci, d_col_idx, (size_t)nnz * sizeof(int), hipMemcpyDeviceToHost, st);
            if (e == hipSuccess && nnz > 0) e = hipMemcpyAsync(val, val_src, (size_t)nnz * sizeof(float), hipMemcpyDeviceToHost, st);
            if (e == hipSuccess) e = hipStreamSynchronize(st);
            if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
            rc = build_streams(rp.data(), ci, val, bp, dp->host, listed_rows);
            if (rc != MPS_OK) return fail(rc);
        }
    } catch (const std::bad_alloc &) {
        return fail(MPS_ERR_UNSUPPORTED);
    }
    Layout &Lo = dp->host;
    if (!on_device) {
        dp->slots = Lo.stream.size() / 2;
        if ((rc = upload(dp, &dp->stream, Lo.stream, st)) != MPS_OK) return fail(rc);
        if (bp_in.keep_src && (rc = upload(dp, &dp->src, Lo.src, st)) != MPS_OK) return fail(rc);
    }
    if ((rc = upload(dp, &dp->panel_ptr, Lo.panel_ptr, st)) != MPS_OK) return fail(rc);
    if ((rc = upload(dp, &dp->rows, Lo.rows, st)) != MPS_OK) return fail(rc);
    if ((rc = upload(dp, &dp->piece_ptr, Lo.piece_ptr, st)) != MPS_OK) return fail(rc);
    if ((rc = upload(dp, &dp->wave_meta, Lo.wave_meta, st)) != MPS_OK) return fail(rc);
    if ((rc = upload(dp, &dp->panel_rounds, Lo.panel_rounds, st)) != MPS_OK) return fail(rc);
    if ((rc = upload(dp, &dp->split_row, Lo.split_row, st)) != MPS_OK) return fail(rc);
    if ((rc = upload(dp, &dp->split_ptr, Lo.split_ptr, st)) != MPS_OK) return fail(rc);
    {
        const size_t bytes = ((size_t)Lo.split_ptr.back() * padded_width(Lo) + 4) * sizeof(float);
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&dp->partial), bytes);
        if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
        dp->device_bytes += bytes;
    }
    dp->lds_bytes = (size_t)(Lo.acc_rows + 1) * Lo.lanes * 16 * (4 / Lo.elem_bytes);
    {
        // the limit belongs to the kernel, not to a plan: always what a CU holds
        hipError_t e = hipSuccess;
        for (const void *kernel : {reinterpret_cast<const void *>(sw_spmm_kernel<float, 4, 1, false>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<float, 4, 1, true>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<float, 4, 2, false>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<float, 4, 2, true>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<float, 8, 1, false>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<float, 8, 1, true>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<float, 8, 2, false>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<float, 8, 2, true>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<half_t, 4, 1, false>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<half_t, 4, 1, true>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<half_t, 4, 2, false>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<half_t, 4, 2, true>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<half_t, 8, 1, false>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<half_t, 8, 1, true>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<half_t, 8, 2, false>),
                                   reinterpret_cast<const void *>(sw_spmm_kernel<half_t, 8, 2, true>)})
            if (e == hipSuccess) e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
    }
    dp->built_on_device = on_device;
    Bulk<uint32_t>().swap(Lo.stream);
    Bulk<int>().swap(Lo.src);
    *out = dp;
    return MPS_OK;
}

int spmm(const DevicePlan *dp, const void *X, void *Y, unsigned phases, hipStream_t st)
{
    if (dp->host.elem_bytes == 4) return spmm_typed<float>(dp, static_cast<const float *>(X), static_cast<float *>(Y), phases, st);
    return spmm_typed<half_t>(dp, static_cast<const half_t *>(X), static_cast<half_t *>(Y), phases, st);
}

int set_values(DevicePlan *dp, const void *d_val, hipStream_t st)
{
    if (!dp->src) return MPS_ERR_UNSUPPORTED;
    if (dp->slots == 0) return MPS_OK;
    const dim3 grid((unsigned)((dp->slots + 255) / 256));
    if (dp->host.elem_bytes == 4)
        hipLaunchKernelGGL((sw_set_values_kernel<float>), grid, dim3(256), 0, st, static_cast<const float *>(d_val), dp->src,
                           dp->slots, dp->stream);
    else
        hipLaunchKernelGGL((sw_set_values_kernel<half_t>), grid, dim3(256), 0, st, static_cast<const half_t *>(d_val), dp->src,
                           dp->slots, dp->stream);
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

const Layout &layout_of(const DevicePlan *dp) { return dp->host; }
bool built_on_device(const DevicePlan *dp) { return dp->built_on_device; }
size_t device_bytes_of(const DevicePlan *dp) { return dp->device_bytes; }

const void *device_array(const DevicePlan *dp, int which, size_t *bytes)
{
    const Layout &Lo = dp->host;
    switch (which) {
    case MPS_PLAN_ARRAY_SW_PANEL_PTR: *bytes = Lo.panel_ptr.size() * sizeof(int); return dp->panel_ptr;
    case MPS_PLAN_ARRAY_SW_ROWS: *bytes = Lo.rows.size() * sizeof(int); return dp->rows;
    case MPS_PLAN_ARRAY_SW_PIECE_PTR: *bytes = Lo.piece_ptr.size() * sizeof(int); return dp->piece_ptr;
    case MPS_PLAN_ARRAY_SW_WAVE_META: *bytes = Lo.wave_meta.size() * sizeof(int); return dp->wave_meta;
    case MPS_PLAN_ARRAY_SW_PANEL_ROUNDS: *bytes = Lo.panel_rounds.size() * sizeof(int); return dp->panel_rounds;
    case MPS_PLAN_ARRAY_SW_STREAM: *bytes = dp->slots * 8; return dp->stream;
    case MPS_PLAN_ARRAY_SW_SRC: *bytes = dp->src ? dp->slots * sizeof(int) : 0; return dp->src;
    case MPS_PLAN_ARRAY_SW_SPLIT_ROW: *bytes = Lo.split_row.size() * sizeof(int); return dp->split_row;
    case MPS_PLAN_ARRAY_SW_SPLIT_PTR: *bytes = Lo.split_ptr.size() * sizeof(int); return dp->split_ptr;
    default: *bytes = 0; return nullptr;
    }
}

}  // namespace mps_sw
