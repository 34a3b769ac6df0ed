// Row-block plans, device side: the kernel that walks the layout of
// mpspmm_rowblock.hpp, and the plan object's device arrays.
//
// Same arithmetic as the reference kernel (src/MergePathSpMM.cu:426-477: one
// fp32 accumulator per output column, a rounded product added per nonzero in
// row order within a run), with explicit values in place of the degree product
// (:450,:459-460); what differs is that the rows of X of the popular columns
// are gathered from LDS, and that a block's output rows are summed in LDS
// instead of through atomics on Y (:445,:477).
#include "mpspmm_device.hpp"
#include "mpspmm_rowblock.hpp"

#include <type_traits>

#include <new>

namespace mps_rb {

struct DevicePlan {
    Layout host;  // the small tables stay filled; the streams are released after the upload
    uint32_t *hot = nullptr;  // the hot stream in packed form (12 bytes per lane and round)
    Entry *cold = nullptr;           // the cold stream as the layout holds it, or
    uint32_t *cold_packed = nullptr;  // in packed form (one of the two)
    int *hot_src = nullptr, *cold_src = nullptr;
    long long *wave_base = nullptr;
    int *meta = nullptr, *block_row = nullptr, *hot_cols = nullptr, *cold_begin = nullptr, *table_base = nullptr, *table_used = nullptr;
    float *hot_x = nullptr;  // [T][H][16] rows of X of the hot columns, gathered per product
    size_t lds_bytes = 0;
    size_t device_bytes = 0;
    size_t hot_slots = 0, cold_slots = 0;
    int keep_from = 0;  // steps from this one on read their streams with plain loads (see kStreamKeepBytes)
    int num_cus = 256;  // CUs the layout was built for: one round of blocks is at most this many
    bool built_on_device = false;
};

namespace {

// hot_x[t][slot][:] = X[hot_cols[t][slot]][:]  (zeros for unused slots)
__global__ __launch_bounds__(256) void rb_gather_hot_kernel(const int *__restrict__ hot_cols,
                                                             const float4 *__restrict__ X4,
                                                             float4 *__restrict__ hot_x4, int slots)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= slots * 4) return;
    const int c = hot_cols[i >> 2];
    hot_x4[i] = c >= 0 ? X4[(size_t)c * 4 + (i & 3)] : make_float4(0.f, 0.f, 0.f, 0.f);
}

constexpr int kThreads = kWaveSlots * 64;
constexpr size_t kStreamKeepBytes = 160u << 20;  // of the entry streams, kept in the last-level cache between products
constexpr int kPrefetch = (kMaxTableRows * 4 + kThreads - 1) / kThreads;  // float4 per thread of one table

// The entry streams are read through buffer descriptors: the base of a wavefront's run of rounds in scalar
// registers, a 32-bit offset per lane, and the cache policy as an operand of the load.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t stream_rsrc(const void *base)
{
    const unsigned long long a = (unsigned long long)base;  // the same in all lanes
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
    return __builtin_amdgcn_make_buffer_rsrc((void *)(((unsigned long long)hi << 32) | lo), 0, 0xffffffff, 0x00020000);
}

// A lane's 16 bytes of a round: its entry of the lane-group's two windows {word A, value A, word B, value B}.
// keep = false: with the streaming hint, which also keeps the line out of the last-level cache; keep = true: a plain
// load, for the part of the streams that is meant to stay there from one product to the next.
__device__ __forceinline__ uint4 load_round(__amdgpu_buffer_rsrc_t r, unsigned off, bool keep)
{
    typedef unsigned u4_t __attribute__((ext_vector_type(4)));
    const u4_t t = keep ? __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0)
                        : __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 2);
    return make_uint4(t[0], t[1], t[2], t[3]);
}

// The same from a packed stream: 12 bytes {value A, value B, half A | half B << 16}, as loaded.  The halves are taken
// apart where the round is used (unpack_round), not here: a round is requested one round ahead, behind the gathers of
// the round before it, and loads return in order - an instruction that touches the loaded words straight away would
// wait for those gathers as well.
__device__ __forceinline__ uint4 load_round_packed(__amdgpu_buffer_rsrc_t r, unsigned off, bool keep)
{
    typedef unsigned u3_t __attribute__((ext_vector_type(3)));
    const u3_t t = keep ? __builtin_amdgcn_raw_buffer_load_b96(r, (int)off, 0, 0)
                        : __builtin_amdgcn_raw_buffer_load_b96(r, (int)off, 0, 2);
    return make_uint4(t[0], t[1], t[2], 0u);
}
__device__ __forceinline__ uint4 unpack_round(const uint4 &t) { return make_uint4(t.z & 0xffffu, t.x, t.z >> 16, t.y); }

// (a value, not a named constant: a float4 object whose address is taken - by a ?: between two lvalues, by a
// reference parameter - is given a private-memory slot of its own and reloaded from there)
__device__ __forceinline__ float4 zero4f() { return make_float4(0.f, 0.f, 0.f, 0.f); }

__device__ __forceinline__ void add4(float4 &a, const float4 &b)
{
    a.x += b.x;
    a.y += b.y;
    a.z += b.z;
    a.w += b.w;
}

// One lane-group's position in one of its two streams.
struct Walk {
    int row;     // block-local row of the nonzeros being summed
    float a[4];  // sums of the current row
};

// Lane j of a lane-group (4 lanes) holds entry j of the group's window.  The other lanes read
// it through a quad permute folded into the instruction that uses it (DPP): no LDS staging, no
// separate move.  A DPP read needs two wait states after a vector-ALU write of its source register,
// and the compiler neither sees a DPP instruction inside an asm statement nor promises where it puts
// the half-word unpack of a packed entry or a register copy.  So every asm statement below begins
// with `s_nop 1` (two wait states) and reads its DPP source only after it: the distance holds by
// construction, whatever wrote the register last.  Outputs are early-clobber: the sources are read
// again further down the same statement.
#define RB_QUAD(j) "quad_perm:[" #j "," #j "," #j "," #j "] row_mask:0xf bank_mask:0xf"
// r[j] = word[lane j of the group] & mask, j = 0 .. N - 1
template <int N>
__device__ __forceinline__ void and_from_lanes(unsigned word, unsigned mask, unsigned (&r)[N])
{
    static_assert(N == 1 || N == 2 || N == 4, "entries of a window that carry a field");
    if constexpr (N == 1)
        asm("s_nop 1\n\tv_and_b32_dpp %0, %1, %2 " RB_QUAD(0) : "=&v"(r[0]) : "v"(word), "v"(mask));
    if constexpr (N == 2)
        asm("s_nop 1\n\tv_and_b32_dpp %0, %2, %3 " RB_QUAD(0) "\n\tv_and_b32_dpp %1, %2, %3 " RB_QUAD(1)
            : "=&v"(r[0]), "=&v"(r[1])
            : "v"(word), "v"(mask));
    if constexpr (N == 4)
        asm("s_nop 1\n\tv_and_b32_dpp %0, %4, %5 " RB_QUAD(0) "\n\tv_and_b32_dpp %1, %4, %5 " RB_QUAD(1)
            "\n\tv_and_b32_dpp %2, %4, %5 " RB_QUAD(2) "\n\tv_and_b32_dpp %3, %4, %5 " RB_QUAD(3)
            : "=&v"(r[0]), "=&v"(r[1]), "=&v"(r[2]), "=&v"(r[3])
            : "v"(word), "v"(mask));
}
// a += val[lane J of the group] * x   (one fused multiply-add per column, as the compiler's fmaf)
template <int J>
__device__ __forceinline__ void fma_from_lane(float (&a)[4], float val, const float4 &x)
{
#define RB_FMAC(j)                                                                                        \
    asm("s_nop 1\n\tv_fmac_f32_dpp %0, %4, %5 " RB_QUAD(j) "\n\tv_fmac_f32_dpp %1, %4, %6 " RB_QUAD(j)    \
        "\n\tv_fmac_f32_dpp %2, %4, %7 " RB_QUAD(j) "\n\tv_fmac_f32_dpp %3, %4, %8 " RB_QUAD(j)           \
        : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3])                                                  \
        : "v"(val), "v"(x.x), "v"(x.y), "v"(x.z), "v"(x.w));
    if constexpr (J == 0) { RB_FMAC(0) }
    if constexpr (J == 1) { RB_FMAC(1) }
    if constexpr (J == 2) { RB_FMAC(2) }
    if constexpr (J == 3) { RB_FMAC(3) }
#undef RB_FMAC
}
#undef RB_QUAD

// rounds (two windows per lane-group each) that a wavefront needs for n windows dealt to its 16 lane-groups
__device__ __forceinline__ int rounds_of(int n) { return ((n >> 4) + ((n & 15) != 0) + 1) >> 1; }

// CPACK: the cold stream is read in its packed form (cold_p; 12 bytes per lane and round, columns counted from the
// first column of the step's range, cold_begin[t]) instead of as 8-byte entries (cold).
template <typename TOut, bool CPACK, bool TABLE_FROM_X>
__global__ __launch_bounds__(kThreads) void rb_spmm_kernel(const uint32_t *__restrict__ hot, const Entry *__restrict__ cold,
                                                            const uint32_t *__restrict__ cold_p,
                                                            const int *__restrict__ cold_begin,
                                                            const long long *__restrict__ wave_base,
                                                            const int4 *__restrict__ meta,
                                                            const int *__restrict__ block_row,
                                                            const float4 *__restrict__ hot_x4,
                                                            const float4 *__restrict__ X4, TOut *__restrict__ Y, int T,
                                                            int H, int acc_rows, int hot_bits, int cold_bits, int keep_from,
                                                            int cold_ib, const int *__restrict__ table_cols,
                                                            const int *__restrict__ table_base,
                                                            const int *__restrict__ table_used, int n_cols)
{
    extern __shared__ __align__(16) char smem[];
    float *table = reinterpret_cast<float *>(smem);                         // [H][16]
    float *acc = table + (size_t)H * 16;                                    // [acc_rows][16]
    float *slots = acc + (size_t)acc_rows * 16;                             // [16 waves][16]
    int *slot_row = reinterpret_cast<int *>(slots + kWaveSlots * 16);       // [16]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 2, s = lane & 3;
    const int b = blockIdx.x;
    float4 *table4 = reinterpret_cast<float4 *>(table);
    float4 *acc4 = reinterpret_cast<float4 *>(acc);
    const int4 *meta_b = meta + (size_t)b * T * kWaveSlots;

    for (int i = tid; i < acc_rows * 4; i += kThreads) acc4[i] = zero4f();
    if (tid < kWaveSlots * 16) slots[tid] = 0.f;
    int local_c0 = 0, local_last = H;  // local tables: the first column of the block's tables, the rows of its last table in use
    if constexpr (TABLE_FROM_X) {
        // the first table straight from X, no gather kernel in front
        if (table_base) {
            // local tables: step t holds the block's own rows c0 + t H .. c0 + (t + 1) H - 1 of X, one contiguous read
            const int c0 = local_c0 = table_base[b];
            local_last = table_used[b];
            const int rows0 = T == 1 ? local_last : H;
            for (int i = tid; i < rows0 * 4; i += kThreads) table4[i] = c0 + (i >> 2) < n_cols ? X4[(size_t)c0 * 4 + i] : zero4f();
        } else {
            for (int i = tid; i < H * 4; i += kThreads) {
                const int c = table_cols[i >> 2];
                table4[i] = c >= 0 ? X4[(size_t)c * 4 + (i & 3)] : zero4f();
            }
        }
    } else {
        for (int i = tid; i < H * 4; i += kThreads) table4[i] = hot_x4[i];
    }

#define RB_PRE_LOAD(k) const float4 pre##k = tid + k * kThreads < pre_lim ? pre_src[tid + k * kThreads] : zero4f();
#define RB_PRE_STORE(k) if (tid + k * kThreads < H * 4) table4[tid + k * kThreads] = pre##k;
    static_assert(kPrefetch == 6, "one RB_PRE_LOAD / RB_PRE_STORE per float4 of a table that a thread moves");

    {
        // ---- every wavefront walks its runs
        long long cur_h = wave_base[((size_t)b * kWaveSlots + wave) * 2];
        long long cur_c = wave_base[((size_t)b * kWaveSlots + wave) * 2 + 1];
        float4 *my_slot4 = reinterpret_cast<float4 *>(slots + wave * 16) + s;
        // the masks live in vector registers (the DPP form of v_and takes no scalar operand); the
        // empty asm keeps the compiler from re-creating them from scalars at every use
        hot_bits = kPackedSlotBits;  // the halves of the packed hot stream: table slot below, a piece of rows_advanced above
        if constexpr (CPACK) cold_bits = cold_ib;  // a 16-bit half: column in the range below, a piece of rows_advanced above
        unsigned hmask = (1u << hot_bits) - 1u, cmask = (1u << cold_bits) - 1u, hot_hi = ~hmask, cold_hi = ~cmask;
        // packed cold windows: entry e holds bits [e p, (e + 1) p) of rows_advanced above the column, p = 16 - cold_ib
        const int cs1 = cold_ib - (16 - cold_ib), cs2 = cold_ib - 2 * (16 - cold_ib), cs3 = cold_ib - 3 * (16 - cold_ib);
        asm volatile("" : "+v"(hmask), "+v"(cmask), "+v"(hot_hi), "+v"(cold_hi));
        int4 m = meta_b[wave];
        // a round of the hot stream: 768 bytes (packed), of the cold stream: 1 KiB
        constexpr unsigned kHotRoundBytes = kPackedRoundWords * 4u;
        constexpr unsigned kColdRoundBytes = CPACK ? kHotRoundBytes : 1024u;
        // A step's streams on their way into L2 before the step is walked: one dword of every 128-byte line (the first
        // 64 lines of each stream: ten rounds), asked for between two walks, where the L1 has nothing else to ask
        // for, with plain loads; the walk then finds its rounds a cache away instead of in HBM, and its own loads of
        // them are the last use.  A wavefront's loads return in order and a line from HBM holds one of the L1's
        // ~64 request slots four to six times as long as a gather that hits L2: asked for during the walk, the
        // stream lines held half of the slot time.  Measured on MI355X, 232,965-row power-law matrix, ms per
        // product: none 0.418; the first 2, 3, 5, 7, 8, 10, 12, 16 rounds of the next step 0.430, 0.421, 0.412,
        // 0.398, 0.393, 0.389, 0.398, 0.398 (a few rounds cost the wait for them and gain little; all rounds of all
        // wavefronts are more than an XCD's L2 holds beside the step's rows of X); with the streaming hint on the
        // requests themselves 0.457; the same ahead of the first step as well: +0.003.
        auto request_ahead = [&](long long at_h, long long at_c, int nh2, int nc2) {
            const int lines_h = min(rounds_of(nh2) * (int)(kHotRoundBytes / 128u), 64);
            const int lines_c = min(rounds_of(nc2) * (int)(kColdRoundBytes / 128u), 64);
            const __amdgpu_buffer_rsrc_t hp2 = stream_rsrc(hot + (size_t)at_h * kPackedRoundWords);
            const __amdgpu_buffer_rsrc_t cp2 = CPACK ? stream_rsrc(cold_p + (size_t)at_c * kPackedRoundWords)
                                                     : stream_rsrc(cold + (size_t)at_c * kRoundEntries);
            unsigned a0 = 0, a1 = 0;
            if (lane < lines_h) a0 = __builtin_amdgcn_raw_buffer_load_b32(hp2, lane * 128, 0, 0);
            if (lane < lines_c) a1 = __builtin_amdgcn_raw_buffer_load_b32(cp2, lane * 128, 0, 0);
            return a0 ^ a1;
        };
        __syncthreads();

        for (int t = 0; t < T; ++t) {
            const int nh = __builtin_amdgcn_readfirstlane(m.x), nc = __builtin_amdgcn_readfirstlane(m.y);
            const int first_row = __builtin_amdgcn_readfirstlane(m.z);
            // next step's counts: in flight while this step is walked
            const int4 m_next = meta_b[(size_t)min(t + 1, T - 1) * kWaveSlots + wave];
            int slot_first = 0;  // wave 0 adds the slots after the barrier: the first rows of all runs of this step
            if (wave == 0) slot_first = meta_b[(size_t)t * kWaveSlots + min(g, kWaves - 1)].z;

            const int rounds_h = rounds_of(nh), rounds_c = rounds_of(nc);
            const int full_h = nh >> 5, full_c = nc >> 5;  // rounds in which every lane-group holds two windows
            const int len_h = (nh >> 4) + (g < (nh & 15)), len_c = (nc >> 4) + (g < (nc & 15));  // windows of this lane-group
            Walk wh, wc;
            wh.row = wc.row = first_row;
#pragma unroll
            for (int i = 0; i < 4; ++i) wh.a[i] = wc.a[i] = 0.f;

            // A window (four nonzeros) lies in one row; its first entry says how many rows the
            // group's run advanced in front of it.  A finished row is added to its LDS
            // accumulator there and then, with a plain read-add-write: among the lane-groups of
            // this wavefront only this one adds to that row while the runs are walked (the others
            // that hold a part of it keep it until after the walk, see tails below), and no other
            // wavefront adds to it directly - except for the first row of the wavefront's run,
            // which goes to the wavefront's slot instead.  (A run's first window counts its rows
            // from the wavefront's first row: the sums that this "row end" adds are zeros.)
            auto row_end = [&](Walk &w, unsigned adv) {
                float4 *dst = w.row == first_row ? my_slot4 : acc4 + (size_t)w.row * 4 + s;
                float4 o = *dst;
                o.x += w.a[0];
                o.y += w.a[1];
                o.z += w.a[2];
                o.w += w.a[3];
                *dst = o;
                w.row += (int)adv;
                w.a[0] = w.a[1] = w.a[2] = w.a[3] = 0.f;
            };
            auto hot_gather = [&](unsigned word, float4 (&x)[kWin]) {
                unsigned slot[kWin];
                and_from_lanes<kWin>(word, hmask, slot);
#pragma unroll
                for (int j = 0; j < kWin; ++j) x[j] = table4[slot[j] * 4 + s];
            };
            // (packed cold entries count their columns from the first column of the step's range)
            const char *xb = reinterpret_cast<const char *>(X4) + (CPACK ? (size_t)cold_begin[t] * 64 : (size_t)0);
            auto cold_gather = [&](unsigned word, float4 (&x)[kWin]) {
                unsigned col[kWin];
                and_from_lanes<kWin>(word, cmask, col);
#pragma unroll
                for (int j = 0; j < kWin; ++j)
                    x[j] = *reinterpret_cast<const float4 *>(xb + (size_t)((col[j] << 6) | (unsigned)(s << 4)));
            };
            // is_hot: a hot window, whose rows_advanced lies in two pieces above the slots of its entries 0 and 1
            // (a packed cold window: in four pieces, one above the column of every entry)
            auto window = [&](auto is_hot, Walk &w, unsigned word, unsigned valbits, const float4 (&x)[kWin], unsigned himask,
                              int bits) {
                if constexpr (decltype(is_hot)::value) {
                    unsigned p[2];
                    and_from_lanes<2>(word, himask, p);
                    if ((p[0] | p[1]) != 0) row_end(w, (p[0] >> kPackedSlotBits) | (p[1] >> (kPackedSlotBits - kPackedPieceBits)));
                } else if constexpr (CPACK) {
                    unsigned p[4];
                    and_from_lanes<4>(word, himask, p);
                    if ((p[0] | p[1] | p[2] | p[3]) != 0) row_end(w, (p[0] >> bits) | (p[1] >> cs1) | (p[2] >> cs2) | (p[3] >> cs3));
                } else {
                    unsigned p[1];
                    and_from_lanes<1>(word, himask, p);
                    if (p[0] != 0) row_end(w, p[0] >> bits);
                }
                const float v = __uint_as_float(valbits);
                fma_from_lane<0>(w.a, v, x[0]);
                fma_from_lane<1>(w.a, v, x[1]);
                fma_from_lane<2>(w.a, v, x[2]);
                fma_from_lane<3>(w.a, v, x[3]);
            };
            // The two windows (A, B) of a round.  have_a / have_b: the lane-group holds them (always, except in
            // the last round of a run).
            auto pair = [&](auto is_hot, Walk &w, const uint4 &cu, const float4 (&xa)[kWin], const float4 (&xb)[kWin],
                            unsigned himask, int bits, bool have_a, bool have_b) {
                if (have_a) window(is_hot, w, cu.x, cu.y, xa, himask, bits);
                if (have_b) window(is_hot, w, cu.z, cu.w, xb, himask, bits);
            };
            constexpr std::true_type kHot{};
            constexpr std::false_type kCold{};

            const bool keep = t >= keep_from;
            const __amdgpu_buffer_rsrc_t hp = stream_rsrc(hot + (size_t)cur_h * kPackedRoundWords);
            const unsigned hoff = (unsigned)lane * 12u;
            auto load_hot = [&](int r) { return load_round_packed(hp, hoff + (unsigned)r * kHotRoundBytes, keep); };
            const __amdgpu_buffer_rsrc_t cp = CPACK ? stream_rsrc(cold_p + (size_t)cur_c * kPackedRoundWords)
                                                    : stream_rsrc(cold + (size_t)cur_c * kRoundEntries);
            const unsigned loff = (unsigned)lane * (CPACK ? 12u : 16u);
            auto load_cold = [&](int r) {
                if constexpr (CPACK) return load_round_packed(cp, loff + (unsigned)r * kColdRoundBytes, keep);
                else return load_round(cp, loff + (unsigned)r * kColdRoundBytes, keep);
            };
            uint4 nx_h = make_uint4(0u, 0u, 0u, 0u), nx_c = nx_h;  // as loaded
            auto take_h = [&]() { return unpack_round(nx_h); };
            auto take_c = [&]() {
                if constexpr (CPACK) return unpack_round(nx_c);
                else return nx_c;
            };
            if (rounds_h > 0) nx_h = load_hot(0);
            if (rounds_c > 0) nx_c = load_cold(0);
            int rh = 0, rc = 0;  // rounds done
            // Round rh / rc has been taken: the next one is requested.  (Two rounds ahead instead of one: 1.5 %
            // slower on the 232,965-row power-law matrix; a round's load is not what the walk waits for.)
            auto advance_h = [&]() {
                ++rh;
                if (rh < rounds_h) nx_h = load_hot(rh);
            };
            auto advance_c = [&]() {
                ++rc;
                if (rc < rounds_c) nx_c = load_cold(rc);
            };
            // The rounds in which every lane-group holds two windows: the hot and the cold ones are
            // spread evenly over max(full_h, full_c) passes (a cold round in every pass whose
            // share of the cold rounds crosses a whole number, likewise for hot), so that the
            // gathers through L2 and the gathers from LDS both run all the time instead of one
            // after the other.
            const int passes = max(full_h, full_c);
            int due_h = (wave * passes) >> 4, due_c = ((wave + 8) * passes) >> 4;  // wavefronts start at different points
            for (int pass = 0; pass < passes; ++pass) {
                // A SIMD serves wavefronts of equal priority oldest first: of the four that share one, the last
                // launched took 40 % longer for the same number of windows (55 against 39 thousand cycles per step
                // on the 232,965-row power-law matrix), and 15 wavefronts waited for it at the barrier.  The
                // priority goes round, a pass at each rank: 46 to 49 thousand cycles for all, the step 7 % shorter.
                // (Since the next step's stream lines are asked for after the walk, equal walks are no longer the aim:
                // a wavefront that is done early has its lines on the way from HBM while the others still gather.
                // Walks by launch rank, thousands of cycles, and ms per product: rank + pass 38 / 34 / 38 / 45 and
                // 0.3835; rank - pass 39 / 37 / 38 / 37 and 0.387 - the evenest and not the fastest; rank + pass + 3,
                // the highest priority to the oldest first, 34 / 42 / 39 / 41 and 0.3807.)
                switch (((wave >> 2) + pass + 3) & 3) {
                case 0: __builtin_amdgcn_s_setprio(0); break;
                case 1: __builtin_amdgcn_s_setprio(1); break;
                case 2: __builtin_amdgcn_s_setprio(2); break;
                default: __builtin_amdgcn_s_setprio(3); break;
                }
                due_h += full_h;
                due_c += full_c;
                const bool do_h = due_h >= passes && rh < full_h, do_c = due_c >= passes && rc < full_c;
                // Both rounds have arrived before anything else is requested.  (Left to the compiler, the wait for the
                // hot round stands where the round is taken apart, behind the cold gathers of this pass: loads return
                // in order, and with a pass that has no cold round in the same code it must assume that nothing was
                // requested after the round - it waits for everything, the gathers included, and the hot round then
                // runs with no gather in flight.)
                asm volatile("" : "+v"(nx_h.z), "+v"(nx_c.z));
                const uint4 cu_c = take_c();
                float4 xca[kWin], xcb[kWin];
                if (do_c) {
                    due_c -= passes;
                    cold_gather(cu_c.x, xca);
                    cold_gather(cu_c.z, xcb);
                    // after the gathers: what waits for them does not wait for this
                    advance_c();
                }
                if (do_h) {
                    due_h -= passes;
                    const uint4 cu_h = take_h();
                    float4 xh[kWin];
                    advance_h();
                    // one window after the other: table rows arrive within a hundred cycles or two, and four rows
                    // in registers instead of eight leave the compiler room (0.3 to 0.6 % faster than both gathered first)
                    hot_gather(cu_h.x, xh);
                    window(kHot, wh, cu_h.x, cu_h.y, xh, hot_hi, 0);
                    hot_gather(cu_h.z, xh);
                    window(kHot, wh, cu_h.z, cu_h.w, xh, hot_hi, 0);
                }
                if (do_c) pair(kCold, wc, cu_c, xca, xcb, cold_hi, cold_bits, true, true);
            }
            // what the rounding of the shares left over
            while (rh < full_h) {
                const uint4 cu_h = take_h();
                float4 xha[kWin], xhb[kWin];
                advance_h();
                hot_gather(cu_h.x, xha);
                hot_gather(cu_h.z, xhb);
                pair(kHot, wh, cu_h, xha, xhb, hot_hi, 0, true, true);
            }
            while (rc < full_c) {
                const uint4 cu_c = take_c();
                float4 xca[kWin], xcb[kWin];
                cold_gather(cu_c.x, xca);
                cold_gather(cu_c.z, xcb);
                advance_c();
                pair(kCold, wc, cu_c, xca, xcb, cold_hi, cold_bits, true, true);
            }
            // the last round of a run: lane-groups hold two, one or none of its windows (the rest is padding)
            if (rc < rounds_c) {
                const uint4 cu_c = take_c();
                float4 xca[kWin], xcb[kWin];
                cold_gather(cu_c.x, xca);
                cold_gather(cu_c.z, xcb);
                pair(kCold, wc, cu_c, xca, xcb, cold_hi, cold_bits, 2 * rc < len_c, 2 * rc + 1 < len_c);
            }
            if (rh < rounds_h) {
                const uint4 cu_h = take_h();
                float4 xha[kWin], xhb[kWin];
                hot_gather(cu_h.x, xha);
                hot_gather(cu_h.z, xhb);
                pair(kHot, wh, cu_h, xha, xhb, hot_hi, 0, 2 * rh < len_h, 2 * rh + 1 < len_h);
            }
            cur_h += rounds_h;
            cur_c += rounds_c;

            // Tails: what every lane-group still holds for the last row of its run.  A group whose
            // neighbours end in other rows adds its sums to the row at once.  Neighbouring groups
            // can also end in the same row (one that is longer than a run): then the first group of
            // the stretch of equal rows gets the stretch's total, summed lane to lane in a fixed
            // tree (no LDS behind it: that space holds table rows), and adds it.
            auto tails = [&](const Walk &w, int len) {
                const int row = len > 0 ? w.row : -1;
                const int prev = __shfl_up(row, 4, 64), next = __shfl_down(row, 4, 64);
                const bool first = g == 0 || prev != row;
                const bool shared = row >= 0 && ((g > 0 && prev == row) || (g < kGroups - 1 && next == row));
                float4 sum = make_float4(w.a[0], w.a[1], w.a[2], w.a[3]);
                if (__any(shared)) {
                    // Sums over 2, 4, 8, 16 neighbouring groups as far as they end in the same row (rows do not
                    // decrease from group to group, so equal rows at distance d mean equal rows in between): after
                    // the four exchanges the first group of a stretch holds the stretch's total.
#pragma unroll
                    for (int d = 1; d < kGroups; d *= 2) {
                        const int there = __shfl_down(row, 4 * d, 64);
                        const float4 v = make_float4(__shfl_down(sum.x, 4 * d, 64), __shfl_down(sum.y, 4 * d, 64),
                                                     __shfl_down(sum.z, 4 * d, 64), __shfl_down(sum.w, 4 * d, 64));
                        if (row >= 0 && g + d < kGroups && there == row) add4(sum, v);
                    }
                }
                if (row >= 0 && first) {
                    float4 *dst = row == first_row ? my_slot4 : acc4 + (size_t)row * 4 + s;
                    float4 o = *dst;
                    add4(o, sum);
                    *dst = o;
                }
            };
            tails(wh, len_h);
            tails(wc, len_c);
            // the next table: on its way while the wavefronts gather at the barrier
            const float4 *pre_src = hot_x4 + (size_t)min(t + 1, T - 1) * H * 4;
            int pre_lim = H * 4;
            if constexpr (TABLE_FROM_X) {
                // local tables: the next H rows of X after this step's, as far as X goes
                const long long first = (long long)local_c0 + (long long)min(t + 1, T - 1) * H;
                pre_src = X4 + first * 4;
                pre_lim = (int)max(0ll, min((long long)(t + 2 >= T ? local_last : H), (long long)n_cols - first)) * 4;
            }
            RB_PRE_LOAD(0) RB_PRE_LOAD(1) RB_PRE_LOAD(2) RB_PRE_LOAD(3) RB_PRE_LOAD(4) RB_PRE_LOAD(5)
            m = m_next;
            // the next step's streams: on their way like the table
            unsigned ahead = 0;
            if (t + 1 < T) ahead = request_ahead(cur_h, cur_c, __builtin_amdgcn_readfirstlane(m.x), __builtin_amdgcn_readfirstlane(m.y));

            __syncthreads();  // every gather from this step's table and every add of this step is done
            if (wave == 0) {
                // Shared rows: slot q holds what wavefront q held back for the first row of its run.
                // Equal rows are adjacent (first rows never decrease); the first lane-group of
                // such a stretch adds its slots in wavefront order.
                const int q = g;
                if (s == 0) slot_row[q] = slot_first;
                wave_lds_sync();
                const bool leader = q < kWaves && (q == 0 || slot_row[q - 1] != slot_first);
                if (leader) {
                    float4 sum = zero4f();
                    for (int k = q; k < kWaves && slot_row[k] == slot_first; ++k)
                        add4(sum, *reinterpret_cast<const float4 *>(slots + k * 16 + s * 4));
                    float4 *dst = acc4 + (size_t)slot_first * 4 + s;
                    float4 o = *dst;
                    add4(o, sum);
                    *dst = o;
                }
                wave_lds_sync();
                *reinterpret_cast<float4 *>(slots + lane * 4) = zero4f();
            }
            if (t + 1 < T) {
                RB_PRE_STORE(0) RB_PRE_STORE(1) RB_PRE_STORE(2) RB_PRE_STORE(3) RB_PRE_STORE(4) RB_PRE_STORE(5)
            }
            __syncthreads();
            asm volatile("" ::"v"(ahead));  // (what keeps the requests: their dwords are of no use)
        }
    }
#undef RB_PRE_LOAD
#undef RB_PRE_STORE

    // the block's rows, once (their range is read here, not held in registers across the walk)
    const int row0 = block_row[b], nrows = block_row[b + 1] - row0;
    for (int i = tid; i < nrows * 4; i += kThreads) {
        const float4 v = acc4[i];
        const float a[4] = {v.x, v.y, v.z, v.w};
        store_acc<4, true>(Y + (size_t)row0 * 16 + (size_t)i * 4, a);
    }
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

template <typename T, typename A>
void release(std::vector<T, A> &v)
{
    std::vector<T, A>().swap(v);
}

// ---------------------------------------------------------------------------------------------------------------
// The builder's passes over the nonzeros, on the device.  The layout is the one that build_layout makes on the host,
// entry for entry: what needs only row_ptr or the nonzero counts of the columns is decided by the same host code
// (plan_blocks, plan_columns), and the kernels below count, cut and place the way passes 1 and 2 of build_layout and
// pack_hot_stream / pack_cold_stream do.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kBuildMaxSteps = 64;  // a wavefront ranks the nonzeros of a row in an LDS table of 2 counters per step

__global__ __launch_bounds__(256) void rbb_degree_kernel(const int *__restrict__ ci, int nnz, int *__restrict__ deg)
{
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < (size_t)nnz; e += (size_t)gridDim.x * blockDim.x)
        atomicAdd(&deg[ci[e]], 1);
}

// One workgroup per row block: range_nnz[r] += the block's nonzeros in column range r of R equal ones; *own += the
// count of its busiest range.
__global__ __launch_bounds__(256) void rbb_ranges_kernel(const int *__restrict__ rp, const int *__restrict__ ci,
                                                          const int *__restrict__ block_row, int n, int R,
                                                          unsigned long long *__restrict__ range_nnz,
                                                          unsigned long long *__restrict__ own)
{
    extern __shared__ int hist[];  // [R], then the block's maximum
    const int b = blockIdx.x, tid = threadIdx.x;
    for (int i = tid; i <= R; i += 256) hist[i] = 0;
    __syncthreads();
    const int e1 = rp[block_row[b + 1]];
    for (int e = rp[block_row[b]] + tid; e < e1; e += 256) atomicAdd(&hist[(int)((long long)ci[e] * R / n)], 1);
    __syncthreads();
    int most = 0;
    for (int i = tid; i < R; i += 256) {
        const int c = hist[i];
        most = max(most, c);
        if (c) atomicAdd(&range_nnz[i], (unsigned long long)c);
    }
    atomicMax(&hist[R], most);
    __syncthreads();
    if (tid == 0) atomicAdd(own, (unsigned long long)hist[R]);
}

// One wavefront per row.  Every nonzero gets its key (step, kind: 0 hot, 1 cold) and its rank among the nonzeros of
// the row with that key, in CSR order.  PLACE false: cnt[((t n) + row) 2 + kind] = nonzeros of the key.  PLACE true:
// the nonzero is written to its place in the packed hot or cold stream (pass 2 of build_layout).
struct PlaceArgs {
    const float *val;
    const int *pre, *prevrow, *block_row, *meta, *run_start, *cuts, *cold_begin;
    const long long *round_off;
    uint32_t *hot, *cold;
    int *hot_src, *cold_src, *overflow;
    int num_blocks, cold_ib;
};

__device__ __forceinline__ void put_entry(uint32_t *stream, int *src, long long round, int g, int e, int which, bool real,
                                          uint32_t value, uint32_t half, int nonzero)
{
    const size_t at = ((size_t)round * 64 + (size_t)(g * kWin + e)) * 3;
    if (real) stream[at + which] = value;
    reinterpret_cast<uint16_t *>(stream + at + 2)[which] = (uint16_t)half;
    if (real && src) src[(size_t)round * kRoundEntries + (size_t)(g * kWin + e) * kPair + which] = nonzero;
}

template <bool PLACE>
__global__ __launch_bounds__(256) void rbb_rows_kernel(const int *__restrict__ rp, const int *__restrict__ ci,
                                                        const int16_t *__restrict__ col_step,
                                                        const int16_t *__restrict__ col_slot, int n, int T, int *cnt,
                                                        PlaceArgs pa)
{
    __shared__ int counters[4][2 * kBuildMaxSteps];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + wave;
    if (r >= n) return;  // (no barrier below: a wavefront works on its own)
    volatile int *base = counters[wave];
    base[lane] = 0;
    base[lane + 64] = 0;
    const int e0 = rp[r], e1 = rp[r + 1];
    int b = 0, lr = 0;
    if constexpr (PLACE) {
        int lo = 0, hi = pa.num_blocks;  // the block of the row: block_row[b] <= r < block_row[b + 1]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (pa.block_row[mid] <= r) lo = mid; else hi = mid;
        }
        b = lo;
        lr = r - pa.block_row[b];
    }
    for (int at = e0; at < e1; at += 64) {
        const int e = at + lane;
        const bool valid = e < e1;
        int c = 0, slot = -1, key = -1;
        if (valid) {
            c = ci[e];
            slot = col_slot[c];
            key = col_step[c] * 2 + (slot < 0);
        }
        int rank = 0;
        unsigned long long todo = __ballot(valid);
        while (todo) {
            const int leader = __ffsll((long long)todo) - 1;
            const int lkey = __shfl(key, leader);
            const bool mine = valid && key == lkey;
            const unsigned long long same = __ballot(mine);
            const int before = base[lkey];
            if (mine) rank = before + __popcll(same & ((1ull << lane) - 1ull));
            if (lane == leader) base[lkey] = before + __popcll(same);
            todo &= ~same;
        }
        if constexpr (PLACE) {
            if (!valid) continue;
            const int t = key >> 1, k = key & 1;
            const size_t gi = ((size_t)t * n + r) * 2;
            const int group = cnt[gi + k];
            const int wi = rank >> 2, en = rank & 3;
            const int pre_h = pa.pre[gi], pre_c = pa.pre[gi + 1];
            const int pk = (k ? pre_c : pre_h) + wi;  // windows of this kind before this one in the step
            const long long q = (long long)pre_h + pre_c + (k ? (cnt[gi] + kWin - 1) / kWin : 0) + wi;  // windows before it
            const size_t bt = (size_t)b * T + t;
            const int *cut = pa.cuts + bt * (kWaves + 1);  // the run of window q: cut[w] <= q < cut[w + 1]
            int w = (int)min(q * kWaves / cut[kWaves], (long long)(kWaves - 1));
            while (w > 0 && q < cut[w]) --w;
            while (q >= cut[w + 1]) ++w;
            const size_t run = bt * kWaveSlots + w;
            int g, j;
            deal(pa.meta[run * 4 + k], pk - pa.run_start[run * 2 + k], &g, &j);
            const int prev = j == 0 ? pa.meta[run * 4 + 2] : (wi > 0 ? lr : pa.prevrow[gi + k]);
            const uint32_t adv = (uint32_t)(lr - prev);
            const long long round = pa.round_off[run * 2 + k] + j / kPair;
            const int which = j % kPair;
            const int pads = rank == group - 1 ? kWin - 1 - en : 0;  // the window's last nonzero repeated with value 0
            const uint32_t value = __float_as_uint(pa.val[e]);
            if (k == 0) {
                if (adv > kPackedAdvMax) *pa.overflow = 1;
                const uint32_t piece_mask = (1u << kPackedPieceBits) - 1u;
                for (int ee = en; ee <= en + pads; ++ee) {
                    const uint32_t piece = ee == 0 ? (adv & piece_mask) : ee == 1 ? ((adv >> kPackedPieceBits) & piece_mask) : 0u;
                    put_entry(pa.hot, pa.hot_src, round, g, ee, which, ee == en, value, (uint32_t)slot | (piece << kPackedSlotBits), e);
                }
            } else {
                const int ib = pa.cold_ib, pb = 16 - ib;
                const uint32_t piece_mask = (1u << pb) - 1u;
                const uint32_t adv_max = pb * kWin >= 32 ? 0xffffffffu : (1u << (pb * kWin)) - 1u;
                const int rel = c - pa.cold_begin[t];
                if (adv > adv_max || rel < 0 || rel >= (1 << ib)) {
                    *pa.overflow = 1;
                    continue;
                }
                for (int ee = en; ee <= en + pads; ++ee)
                    put_entry(pa.cold, pa.cold_src, round, g, ee, which, ee == en, value,
                              (uint32_t)rel | (((adv >> (pb * ee)) & piece_mask) << ib), e);
            }
        }
    }
    if constexpr (!PLACE)
        for (int key = lane; key < 2 * T; key += 64) cnt[((size_t)(key >> 1) * n + r) * 2 + (key & 1)] = base[key];
}

// Exclusive sums and exclusive maxima over the 1,024 threads of a workgroup (scratch: 17 ints of LDS).
__device__ __forceinline__ int block_sum_before(int v, int *total, int *scratch)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = v;
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(inc, d);
        if (lane >= d) inc += o;
    }
    if (lane == 63) scratch[wave] = inc;
    __syncthreads();
    if (wave == 0) {
        const int s = lane < 16 ? scratch[lane] : 0;
        int si = s;
        for (int d = 1; d < 16; d <<= 1) {
            const int o = __shfl_up(si, d);
            if (lane >= d) si += o;
        }
        if (lane < 16) scratch[lane] = si - s;
        if (lane == 15) scratch[16] = si;
    }
    __syncthreads();
    const int before = inc - v + scratch[wave];
    *total = scratch[16];
    __syncthreads();
    return before;
}

__device__ __forceinline__ int block_max_before(int v, int *scratch)  // -1 where nothing comes before
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = v;
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(inc, d);
        if (lane >= d) inc = max(inc, o);
    }
    if (lane == 63) scratch[wave] = inc;
    __syncthreads();
    if (wave == 0) {
        int si = lane < 16 ? scratch[lane] : -1;
        for (int d = 1; d < 16; d <<= 1) {
            const int o = __shfl_up(si, d);
            if (lane >= d) si = max(si, o);
        }
        const int ex = __shfl_up(si, 1);
        if (lane < 16) scratch[lane] = lane == 0 ? -1 : ex;
    }
    __syncthreads();
    const int up = __shfl_up(inc, 1);
    const int before = max(lane == 0 ? -1 : up, scratch[wave]);
    __syncthreads();
    return before;
}

// One workgroup per (block, step), one thread per row of the block (pass 1 of build_layout, split_step): the windows
// of kind k before every row (pre), the last row before it that has any (prevrow), the 16 runs (meta: {hot windows,
// cold windows, first row, 0}; run_start: hot and cold windows of the step before the run; cuts: all windows of the
// step before the run, and the step's windows in all as the 17th).
__global__ __launch_bounds__(1024) void rbb_split_kernel(const int *__restrict__ cnt, const int *__restrict__ block_row, int n,
                                                          int T, int *__restrict__ pre, int *__restrict__ prevrow,
                                                          int *__restrict__ meta, int *__restrict__ run_start,
                                                          int *__restrict__ cuts)
{
    __shared__ int scratch[17], first_row[kWaves], hstart[kWaves + 1], cstart[kWaves + 1], cut[kWaves + 1];
    __shared__ unsigned long long best;
    const int b = blockIdx.x / T, t = blockIdx.x % T, lr = threadIdx.x;
    const int r0 = block_row[b], nr = block_row[b + 1] - r0;
    const size_t gi = ((size_t)t * n + (size_t)(r0 + lr)) * 2;
    int h = 0, c = 0;
    if (lr < nr) {
        h = (cnt[gi] + kWin - 1) / kWin;
        c = (cnt[gi + 1] + kWin - 1) / kWin;
    }
    int hot_total, cold_total;
    const int hq = block_sum_before(h, &hot_total, scratch), cq = block_sum_before(c, &cold_total, scratch);
    const int ph = block_max_before(h > 0 ? lr : -1, scratch), pc = block_max_before(c > 0 ? lr : -1, scratch);
    if (lr < nr) {
        pre[gi] = hq;
        pre[gi + 1] = cq;
        prevrow[gi] = ph;
        prevrow[gi + 1] = pc;
    }
    if (lr <= kWaves) {  // a step without windows: every run begins and ends at 0
        if (lr < kWaves) first_row[lr] = 0;
        hstart[lr] = lr < kWaves ? 0 : hot_total;
        cstart[lr] = lr < kWaves ? 0 : cold_total;
        cut[lr] = lr < kWaves ? 0 : hot_total + cold_total;
    }
    __syncthreads();
    // The cuts one after the other, as split_step makes them: every row looks at the places for the cut that lie
    // among its own windows, the best key wins.
    const long long E = (long long)hot_total + cold_total, q0 = (long long)hq + cq;
    const long long slack = E / kWaves / kCutSlack;
    for (int w = E > 0 ? 0 : kWaves; w < kWaves; ++w) {
        const long long equal_cut = (long long)w * E / kWaves;
        const long long lo = w == 0 ? 0 : max((long long)cut[w - 1], equal_cut - slack);
        const long long hi = w == 0 ? 0 : min(equal_cut + slack, E - 1);
        const int run_h = w == 0 ? 0 : hstart[w - 1], run_c = w == 0 ? 0 : cstart[w - 1];
        if (lr == 0) best = ~0ull;
        __syncthreads();
        unsigned long long mine = ~0ull;
        for (long long q = max(lo, q0); q <= min(hi, q0 + h + c - 1); ++q) {
            const long long d = q - q0;
            const int hot = d < h ? hq + (int)d : hq + h, cold = d < h ? cq : cq + (int)(d - h);
            mine = min(mine, cut_key(hot - run_h, cold - run_c, q, equal_cut));
        }
        if (mine != ~0ull) atomicMin(&best, mine);
        __syncthreads();
        const long long q = (long long)(best & 0xffffffffull);
        if (q >= q0 && q < q0 + h + c) {  // the row that holds the cut
            const long long d = q - q0;
            cut[w] = (int)q;
            first_row[w] = lr;
            hstart[w] = d < h ? hq + (int)d : hq + h;
            cstart[w] = d < h ? cq : cq + (int)(d - h);
        }
        __syncthreads();
    }
    const size_t bt = (size_t)b * T + t;
    if (lr < kWaves) {
        int *m = meta + (bt * kWaveSlots + lr) * 4;
        m[0] = hstart[lr + 1] - hstart[lr];
        m[1] = cstart[lr + 1] - cstart[lr];
        m[2] = first_row[lr];
        m[3] = 0;
        run_start[(bt * kWaveSlots + lr) * 2] = hstart[lr];
        run_start[(bt * kWaveSlots + lr) * 2 + 1] = cstart[lr];
    }
    if (lr <= kWaves) cuts[bt * (kWaves + 1) + lr] = cut[lr];
}

// Device memory that lives for the length of a build
struct Scratch {
    void *p = nullptr;
    ~Scratch()
    {
        if (p) (void)hipFree(p);
    }
    hipError_t get(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 4); }
    template <typename T>
    T *as() const
    {
        return static_cast<T *>(p);
    }
};

#define RBB_TRY(expr)                                           \
    do {                                                        \
        const hipError_t e_ = (expr);                           \
        if (e_ != hipSuccess) return MPS_ERR_HIP + (int)e_;     \
    } while (0)

// Builds the layout with the passes over the nonzeros on the device.  The streams end up in dp's device arrays, the
// small tables in dp->host as after build_layout.  kNeedHost: this matrix is for the host builder (local tables,
// more than kBuildMaxSteps steps, a cold stream that cannot be packed); nothing of dp is to be kept then.
int build_on_device(const int *d_rp, const int *d_ci, const float *d_val, int n, int nnz, const BuildParams &bp, hipStream_t st,
                    DevicePlan *dp)
{
    Layout &L = dp->host;
    std::vector<int> rp((size_t)n + 1);
    RBB_TRY(hipMemcpyAsync(rp.data(), d_rp, ((size_t)n + 1) * sizeof(int), hipMemcpyDeviceToHost, st));
    RBB_TRY(hipStreamSynchronize(st));
    if (rp[0] != 0 || rp[(size_t)n] != nnz) return MPS_ERR_INVALID_CSR;
    int H = 0;
    int rc = plan_blocks(rp.data(), n, nnz, bp, L, &H);
    if (rc != MPS_OK) return rc;
    const int NB = L.num_blocks;
    if ((rc = upload(dp, &dp->block_row, L.block_row, st)) != MPS_OK) return rc;

    // nonzeros per column
    Scratch d_deg;
    RBB_TRY(d_deg.get((size_t)n * sizeof(int)));
    RBB_TRY(hipMemsetAsync(d_deg.p, 0, (size_t)n * sizeof(int), st));
    if (nnz > 0)
        hipLaunchKernelGGL(rbb_degree_kernel, dim3((unsigned)std::min<long long>(((long long)nnz + 255) / 256, 8192)), dim3(256), 0,
                           st, d_ci, nnz, d_deg.as<int>());
    std::vector<int> deg((size_t)n);
    RBB_TRY(hipMemcpyAsync(deg.data(), d_deg.p, (size_t)n * sizeof(int), hipMemcpyDeviceToHost, st));
    RBB_TRY(hipStreamSynchronize(st));
    int failed = MPS_OK;
    auto block_ranges = [&](int R, long long *own, long long *busiest) {
        *own = *busiest = 0;
        Scratch d_ranges;
        std::vector<unsigned long long> ranges((size_t)R + 1, 0ull);
        hipError_t e = d_ranges.get(ranges.size() * sizeof(unsigned long long));
        if (e == hipSuccess) e = hipMemsetAsync(d_ranges.p, 0, ranges.size() * sizeof(unsigned long long), st);
        if (e == hipSuccess) {
            hipLaunchKernelGGL(rbb_ranges_kernel, dim3((unsigned)NB), dim3(256), ((size_t)R + 1) * sizeof(int), st, d_rp, d_ci,
                               dp->block_row, n, R, d_ranges.as<unsigned long long>(), d_ranges.as<unsigned long long>() + R);
            e = hipMemcpyAsync(ranges.data(), d_ranges.p, ranges.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost, st);
        }
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) {
            failed = MPS_ERR_HIP + (int)e;
            return;
        }
        *own = (long long)ranges[(size_t)R];
        for (int r = 0; r < R; ++r) *busiest = std::max(*busiest, (long long)ranges[(size_t)r]);
    };
    ColumnMap cm;
    rc = plan_columns(rp.data(), nullptr, n, nnz, bp, L, H, deg.data(), block_ranges, cm);
    if (failed != MPS_OK) return failed;
    if (rc != MPS_OK) return rc;
    const int T = L.steps;
    if (T > kBuildMaxSteps || (size_t)T * (size_t)n * 2 * sizeof(int) > ((size_t)512 << 20)) return kNeedHost;
    if (L.hot_bits > kPackedSlotBits) return MPS_ERR_UNSUPPORTED;
    int widest = 1;
    for (int t = 0; t < T; ++t) widest = std::max(widest, L.cold_begin[(size_t)t + 1] - L.cold_begin[(size_t)t]);
    const int ib = std::max(12, bits_for(widest > 1 ? widest - 1 : 1));
    if (ib > 15) return kNeedHost;

    // passes 1 and 2
    Scratch d_step, d_slot, d_cnt, d_pre, d_prev, d_run_start, d_cuts, d_round_off, d_flag;
    const size_t groups = (size_t)T * (size_t)n * 2, runs = (size_t)NB * T * kWaveSlots;
    RBB_TRY(d_step.get((size_t)n * sizeof(int16_t)));
    RBB_TRY(d_slot.get((size_t)n * sizeof(int16_t)));
    RBB_TRY(d_cnt.get(groups * sizeof(int)));
    RBB_TRY(d_pre.get(groups * sizeof(int)));
    RBB_TRY(d_prev.get(groups * sizeof(int)));
    RBB_TRY(d_run_start.get(runs * 2 * sizeof(int)));
    RBB_TRY(d_cuts.get((size_t)NB * T * (kWaves + 1) * sizeof(int)));
    RBB_TRY(d_round_off.get(runs * 2 * sizeof(long long)));
    RBB_TRY(d_flag.get(sizeof(int)));
    RBB_TRY(hipMemcpyAsync(d_step.p, cm.step.data(), (size_t)n * sizeof(int16_t), hipMemcpyHostToDevice, st));
    RBB_TRY(hipMemcpyAsync(d_slot.p, cm.slot.data(), (size_t)n * sizeof(int16_t), hipMemcpyHostToDevice, st));
    RBB_TRY(hipMemsetAsync(d_flag.p, 0, sizeof(int), st));
    if ((rc = upload(dp, &dp->cold_begin, L.cold_begin, st)) != MPS_OK) return rc;
    RBB_TRY(hipMalloc(reinterpret_cast<void **>(&dp->meta), runs * 4 * sizeof(int)));
    dp->device_bytes += runs * 4 * sizeof(int);
    const dim3 row_grid((unsigned)((n + 3) / 4));
    PlaceArgs pa{};
    hipLaunchKernelGGL(rbb_rows_kernel<false>, row_grid, dim3(256), 0, st, d_rp, d_ci, d_step.as<int16_t>(), d_slot.as<int16_t>(), n,
                       T, d_cnt.as<int>(), pa);
    hipLaunchKernelGGL(rbb_split_kernel, dim3((unsigned)(NB * T)), dim3(1024), 0, st, d_cnt.as<int>(), dp->block_row, n, T,
                       d_pre.as<int>(), d_prev.as<int>(), dp->meta, d_run_start.as<int>(), d_cuts.as<int>());
    L.meta.resize(runs * 4);
    RBB_TRY(hipMemcpyAsync(L.meta.data(), dp->meta, runs * 4 * sizeof(int), hipMemcpyDeviceToHost, st));
    RBB_TRY(hipStreamSynchronize(st));
    // where every wavefront's streams start, and where it stands at the start of every step
    std::vector<long long> round_off(runs * 2);
    L.wave_base.assign((size_t)NB * kWaveSlots * 2, 0);
    long long hr = 0, cr = 0;
    for (int b = 0; b < NB; ++b)
        for (int w = 0; w < kWaveSlots; ++w) {
            L.wave_base[((size_t)b * kWaveSlots + w) * 2] = hr;
            L.wave_base[((size_t)b * kWaveSlots + w) * 2 + 1] = cr;
            for (int t = 0; t < T; ++t) {
                const size_t run = ((size_t)b * T + t) * kWaveSlots + w;
                round_off[run * 2] = hr;
                round_off[run * 2 + 1] = cr;
                hr += rounds_for(L.meta[run * 4]);
                cr += rounds_for(L.meta[run * 4 + 1]);
            }
        }
    L.hot_rounds = hr;
    L.cold_rounds = cr;
    L.cold_index_bits = ib;
    RBB_TRY(hipMemcpyAsync(d_round_off.p, round_off.data(), round_off.size() * sizeof(long long), hipMemcpyHostToDevice, st));
    if ((rc = upload(dp, &dp->wave_base, L.wave_base, st)) != MPS_OK) return rc;
    const size_t hot_bytes = (size_t)hr * kPackedRoundWords * sizeof(uint32_t), cold_bytes = (size_t)cr * kPackedRoundWords * sizeof(uint32_t);
    RBB_TRY(hipMalloc(reinterpret_cast<void **>(&dp->hot), hot_bytes ? hot_bytes : 4));
    if (cold_bytes) {
        RBB_TRY(hipMalloc(reinterpret_cast<void **>(&dp->cold_packed), cold_bytes));
        RBB_TRY(hipMemsetAsync(dp->cold_packed, 0, cold_bytes, st));
    } else {  // (no cold entries: like the host builder's plan, which then holds an empty unpacked stream)
        RBB_TRY(hipMalloc(reinterpret_cast<void **>(&dp->cold), sizeof(Entry)));
    }
    dp->device_bytes += (hot_bytes ? hot_bytes : 4) + (cold_bytes ? cold_bytes : sizeof(Entry));
    RBB_TRY(hipMemsetAsync(dp->hot, 0, hot_bytes, st));
    if (bp.keep_src) {
        const size_t hs = (size_t)hr * kRoundEntries * sizeof(int), cs = (size_t)cr * kRoundEntries * sizeof(int);
        RBB_TRY(hipMalloc(reinterpret_cast<void **>(&dp->hot_src), hs ? hs : 4));
        RBB_TRY(hipMalloc(reinterpret_cast<void **>(&dp->cold_src), cs ? cs : 4));
        dp->device_bytes += (hs ? hs : 4) + (cs ? cs : 4);
        RBB_TRY(hipMemsetAsync(dp->hot_src, 0xff, hs, st));
        RBB_TRY(hipMemsetAsync(dp->cold_src, 0xff, cs, st));
    }
    pa.val = d_val;
    pa.pre = d_pre.as<int>();
    pa.prevrow = d_prev.as<int>();
    pa.block_row = dp->block_row;
    pa.meta = dp->meta;
    pa.run_start = d_run_start.as<int>();
    pa.cuts = d_cuts.as<int>();
    pa.cold_begin = dp->cold_begin;
    pa.round_off = d_round_off.as<long long>();
    pa.hot = dp->hot;
    pa.cold = dp->cold_packed;
    pa.hot_src = dp->hot_src;
    pa.cold_src = dp->cold_src;
    pa.overflow = d_flag.as<int>();
    pa.num_blocks = NB;
    pa.cold_ib = ib;
    hipLaunchKernelGGL(rbb_rows_kernel<true>, row_grid, dim3(256), 0, st, d_rp, d_ci, d_step.as<int16_t>(), d_slot.as<int16_t>(), n,
                       T, d_cnt.as<int>(), pa);
    RBB_TRY(hipGetLastError());
    int overflow = 0;
    RBB_TRY(hipMemcpyAsync(&overflow, d_flag.p, sizeof(int), hipMemcpyDeviceToHost, st));
    RBB_TRY(hipStreamSynchronize(st));
    if (overflow) return kNeedHost;  // a window advances more rows than the packed forms hold
    return MPS_OK;
}
#undef RBB_TRY

}  // namespace

void destroy(DevicePlan *dp)
{
    if (!dp) return;
    (void)hipFree(dp->hot);
    (void)hipFree(dp->cold);
    (void)hipFree(dp->cold_packed);
    (void)hipFree(dp->cold_begin);
    (void)hipFree(dp->table_base);
    (void)hipFree(dp->table_used);
    (void)hipFree(dp->hot_src);
    (void)hipFree(dp->cold_src);
    (void)hipFree(dp->wave_base);
    (void)hipFree(dp->meta);
    (void)hipFree(dp->block_row);
    (void)hipFree(dp->hot_cols);
    (void)hipFree(dp->hot_x);
    delete dp;
}

// Builds the layout - with the passes over the nonzeros on the device where build_on_device takes the matrix, else
// from a copy of the CSR arrays on the host - and uploads what is not on the device yet.  The arrays must have passed
// mps_csr_validate.
int create(const int *d_row_ptr, const int *d_col_idx, const float *d_val, int n, int nnz, int K, const BuildParams &bp_in,
           hipStream_t st, DevicePlan **out)
{
    *out = nullptr;
    DevicePlan *dp = new (std::nothrow) DevicePlan;
    if (!dp) return MPS_ERR_UNSUPPORTED;
    int rc = MPS_OK;
    auto fail = [&](int code) {
        (void)hipStreamSynchronize(st);  // uploads from the layout's host arrays may still be in flight
        destroy(dp);
        return code;
    };
    bool on_device = false;
    try {
        BuildParams bp = bp_in;
        if (bp.num_cus <= 0) {
            int dev = 0, cus = 256;
            hipError_t e = hipGetDevice(&dev);
            if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
            bp.num_cus = cus;
        }
        if (K != 16) return fail(MPS_ERR_UNSUPPORTED);
        dp->num_cus = bp.num_cus;
        if (!bp.host_build) {
            rc = build_on_device(d_row_ptr, d_col_idx, d_val, n, nnz, bp, st, dp);
            if (rc == MPS_OK) {
                on_device = true;
            } else {
                // start again from an empty plan: for another error than kNeedHost, to give it back
                (void)hipStreamSynchronize(st);
                destroy(dp);
                dp = nullptr;
                // (the device passes need room beside the matrix for their counts and ranks: without it, the host's)
                if (rc == MPS_ERR_HIP + (int)hipErrorOutOfMemory) {
                    (void)hipGetLastError();
                    rc = kNeedHost;
                }
                if (rc != kNeedHost) return rc;
                dp = new (std::nothrow) DevicePlan;
                if (!dp) return MPS_ERR_UNSUPPORTED;
                dp->num_cus = bp.num_cus;
            }
        }
        if (!on_device) {
            // The CSR arrays come back into pinned host memory (a pageable target takes ten times as long: 0.27 s
            // against 0.02 s per GiB on MI355X hosts) and are released as soon as the layout is built.
            struct Pinned {
                void *p = nullptr;
                ~Pinned() { if (p) (void)hipHostFree(p); }
            } h_rp, h_ci, h_val;
            hipError_t e = hipHostMalloc(&h_rp.p, ((size_t)n + 1) * sizeof(int), hipHostMallocDefault);
            if (e == hipSuccess) e = hipHostMalloc(&h_ci.p, ((size_t)nnz + 1) * sizeof(int), hipHostMallocDefault);
            if (e == hipSuccess) e = hipHostMalloc(&h_val.p, ((size_t)nnz + 1) * sizeof(float), hipHostMallocDefault);
            if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
            int *rp = static_cast<int *>(h_rp.p), *ci = static_cast<int *>(h_ci.p);
            float *val = static_cast<float *>(h_val.p);
            e = hipMemcpyAsync(rp, d_row_ptr, ((size_t)n + 1) * sizeof(int), hipMemcpyDeviceToHost, st);
            if (e == hipSuccess && nnz > 0) e = hipMemcpyAsync(ci, d_col_idx, (size_t)nnz * sizeof(int), hipMemcpyDeviceToHost, st);
            if (e == hipSuccess && nnz > 0) e = hipMemcpyAsync(val, d_val, (size_t)nnz * sizeof(float), hipMemcpyDeviceToHost, st);
            if (e == hipSuccess) e = hipStreamSynchronize(st);
            if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
            // (the caller has run mps_csr_validate on the device arrays: the builder indexes by column id)
            if (rp[0] != 0 || rp[(size_t)n] != nnz) return fail(MPS_ERR_INVALID_CSR);
            rc = build_layout(rp, ci, val, n, nnz, K, bp, dp->host);
            if (rc != MPS_OK) return fail(rc);
        }
    } catch (const std::bad_alloc &) {
        return fail(MPS_ERR_UNSUPPORTED);
    }
    Layout &L = dp->host;
    dp->hot_slots = (size_t)L.hot_rounds * kRoundEntries;
    dp->cold_slots = (size_t)L.cold_rounds * kRoundEntries;
    const bool cold_is_packed = on_device ? dp->cold_packed != nullptr : !L.cold_packed.empty();
    {
        // Streams that fit the 256 MiB last-level cache (kStreamKeepBytes of them, from the last step backwards) are
        // read with plain loads and so stay there from one product to the next; all others carry the streaming hint
        // and pass it by.  A product reads a plan once, front to back: left to itself the cache would hold the end of
        // the previous pass and lose it again before the next pass gets there.  Streams of more than twice that size
        // are not kept at all: every step's lines are asked for ahead of its walk (request_ahead in the kernel), which
        // serves the walk better than a cache that holds a fifth of them.  Measured on MI355X, ms per product, no
        // step kept against kStreamKeepBytes kept: 232,965-row power-law matrix with 115 M nonzeros (803 MB of
        // streams, 3 of 16 steps) 0.385 / 0.390; with 50 M nonzeros (351 MB) 0.2165 / 0.2163; with 20 M (140 MB, all
        // kept) 0.1218 / 0.1184; R-MAT scale 20 (130 MB, all kept) 0.194 / 0.187.  (Before the lines were asked for
        // ahead, the 115 M-nonzero matrix ran at 0.435, 0.4285, 0.432, 0.442 ms with 2, 3, 4, 5 steps kept.)
        const size_t hot_bytes = (size_t)L.hot_rounds * kPackedRoundWords * sizeof(uint32_t);
        const size_t cold_bytes = cold_is_packed ? (size_t)L.cold_rounds * kPackedRoundWords * sizeof(uint32_t) : dp->cold_slots * sizeof(Entry);
        const size_t per_step = (hot_bytes + cold_bytes) / (size_t)(L.steps > 0 ? L.steps : 1);
        size_t keep = per_step > 0 ? kStreamKeepBytes / per_step : (size_t)L.steps;
        if (hot_bytes + cold_bytes > 2 * kStreamKeepBytes) keep = 0;
        dp->keep_from = keep >= (size_t)L.steps ? 0 : L.steps - (int)keep;
    }
    if (!on_device) {
        if ((rc = upload(dp, &dp->hot, L.hot_packed, st)) != MPS_OK) return fail(rc);
        if (L.cold_packed.empty()) {
            if ((rc = upload(dp, &dp->cold, L.cold, st)) != MPS_OK) return fail(rc);
        } else if ((rc = upload(dp, &dp->cold_packed, L.cold_packed, st)) != MPS_OK) {
            return fail(rc);
        }
        if ((rc = upload(dp, &dp->cold_begin, L.cold_begin, st)) != MPS_OK) return fail(rc);
        if (!L.table_base.empty() && (rc = upload(dp, &dp->table_base, L.table_base, st)) != MPS_OK) return fail(rc);
        if (!L.table_used.empty() && (rc = upload(dp, &dp->table_used, L.table_used, st)) != MPS_OK) return fail(rc);
        if (bp_in.keep_src) {
            if ((rc = upload(dp, &dp->hot_src, L.hot_src, st)) != MPS_OK) return fail(rc);
            if ((rc = upload(dp, &dp->cold_src, L.cold_src, st)) != MPS_OK) return fail(rc);
        }
        if ((rc = upload(dp, &dp->wave_base, L.wave_base, st)) != MPS_OK) return fail(rc);
        if ((rc = upload(dp, &dp->meta, L.meta, st)) != MPS_OK) return fail(rc);
        if ((rc = upload(dp, &dp->block_row, L.block_row, st)) != MPS_OK) return fail(rc);
    }
    if ((rc = upload(dp, &dp->hot_cols, L.hot_cols, st)) != MPS_OK) return fail(rc);
    {
        const size_t bytes = (size_t)L.steps * L.table_rows * 16 * sizeof(float);
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&dp->hot_x), bytes);
        if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
        dp->device_bytes += bytes;
    }
    dp->lds_bytes = (size_t)(L.table_rows + L.acc_rows) * 64 + kSlotBytes;
    {
        // The dynamic-LDS limit of a kernel is one value per kernel, not per plan: it is set to the most any plan
        // can ask for (kLdsBytes), never to this plan's own size, so that a later plan with a smaller table
        // cannot lower it under an earlier plan that is still in use.
        hipError_t e = hipSuccess;
        for (const void *kernel : {reinterpret_cast<const void *>(rb_spmm_kernel<float, false, false>),
                                   reinterpret_cast<const void *>(rb_spmm_kernel<float, true, false>),
                                   reinterpret_cast<const void *>(rb_spmm_kernel<float, false, true>),
                                   reinterpret_cast<const void *>(rb_spmm_kernel<float, true, true>)})
            if (e == hipSuccess) e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) return fail(MPS_ERR_HIP + (int)e);
    }
    dp->built_on_device = on_device;
    release(L.hot);
    release(L.hot_packed);
    release(L.cold);
    release(L.cold_packed);
    release(L.hot_src);
    release(L.cold_src);
    *out = dp;
    return MPS_OK;
}

int spmm(const DevicePlan *dp, const float *X, float *Y, unsigned phases, hipStream_t st)
{
    const Layout &L = dp->host;
    const int slots = L.steps * L.table_rows;
    // A plan of one step and one round of blocks loads its table from X in the main kernel: a launch less (4,096 rows
    // x 8 per row: 9.4 against 11.2 us per product).  With more blocks than CUs the gathers of every block cost more
    // than the launch (R-MAT scale 18 x 16, 512 blocks: 50 against 46 us).
    // Local tables differ from block to block and are contiguous in X: always read there.
    const bool table_from_x = (L.steps == 1 && L.num_blocks <= dp->num_cus) || dp->table_base;
    if ((phases & MPS_PHASE_PREPARE) && !table_from_x)
        hipLaunchKernelGGL(rb_gather_hot_kernel, dim3((unsigned)((slots * 4 + 255) / 256)), dim3(256), 0, st, dp->hot_cols,
                           reinterpret_cast<const float4 *>(X), reinterpret_cast<float4 *>(dp->hot_x), slots);
    if (phases & MPS_PHASE_MAIN) {
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, dim3((unsigned)L.num_blocks), dim3(kThreads), dp->lds_bytes, st, dp->hot, dp->cold,
                               dp->cold_packed, dp->cold_begin, dp->wave_base, reinterpret_cast<const int4 *>(dp->meta),
                               dp->block_row, reinterpret_cast<const float4 *>(dp->hot_x), reinterpret_cast<const float4 *>(X),
                               Y, L.steps, L.table_rows, L.acc_rows, L.hot_bits, L.cold_bits, dp->keep_from, L.cold_index_bits,
                               table_from_x ? dp->hot_cols : nullptr, dp->table_base, dp->table_used, L.n);
        };
        if (table_from_x) {
            if (dp->cold_packed) launch(rb_spmm_kernel<float, true, true>);
            else launch(rb_spmm_kernel<float, false, true>);
        } else if (dp->cold_packed) {
            launch(rb_spmm_kernel<float, true, false>);
        } else {
            launch(rb_spmm_kernel<float, false, false>);
        }
    }
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

namespace {
__global__ __launch_bounds__(256) void rb_set_values_kernel(const float *__restrict__ val, const int *__restrict__ src,
                                                             size_t slots, Entry *__restrict__ entries)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= slots) return;
    const int e = src[i];
    if (e >= 0) entries[i].val = val[e];
}

// The same for a packed stream: entry slot i is value (i % 2) of lane (i % 128) / 2 of round i / 128.
__global__ __launch_bounds__(256) void rb_set_values_packed_kernel(const float *__restrict__ val,
                                                                    const int *__restrict__ src, size_t slots,
                                                                    uint32_t *__restrict__ packed)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= slots) return;
    const int e = src[i];
    if (e < 0) return;
    const size_t round = i / kRoundEntries, within = i % kRoundEntries;
    packed[(round * 64 + within / kPair) * 3 + within % kPair] = __float_as_uint(val[e]);
}
}  // namespace

int set_values(DevicePlan *dp, const float *d_val, hipStream_t st)
{
    if (!dp->hot_src || !dp->cold_src) return MPS_ERR_UNSUPPORTED;
    if (dp->hot_slots)
        hipLaunchKernelGGL(rb_set_values_packed_kernel, dim3((unsigned)((dp->hot_slots + 255) / 256)), dim3(256), 0, st, d_val,
                           dp->hot_src, dp->hot_slots, dp->hot);
    if (dp->cold_slots && dp->cold_packed)
        hipLaunchKernelGGL(rb_set_values_packed_kernel, dim3((unsigned)((dp->cold_slots + 255) / 256)), dim3(256), 0, st, d_val,
                           dp->cold_src, dp->cold_slots, dp->cold_packed);
    else if (dp->cold_slots)
        hipLaunchKernelGGL(rb_set_values_kernel, dim3((unsigned)((dp->cold_slots + 255) / 256)), dim3(256), 0, st, d_val,
                           dp->cold_src, dp->cold_slots, dp->cold);
    MPS_HIP_TRY(hipGetLastError());
    return MPS_OK;
}

const Layout &layout_of(const DevicePlan *dp) { return dp->host; }
bool built_on_device(const DevicePlan *dp) { return dp->built_on_device; }

const void *device_array(const DevicePlan *dp, int which, size_t *bytes)
{
    const Layout &L = dp->host;
    switch (which) {
    case MPS_PLAN_ARRAY_RB_BLOCK_ROW: *bytes = L.block_row.size() * sizeof(int); return dp->block_row;
    case MPS_PLAN_ARRAY_RB_HOT_COLS: *bytes = L.hot_cols.size() * sizeof(int); return dp->hot_cols;
    case MPS_PLAN_ARRAY_RB_META: *bytes = L.meta.size() * sizeof(int); return dp->meta;
    case MPS_PLAN_ARRAY_RB_WAVE_BASE: *bytes = L.wave_base.size() * sizeof(long long); return dp->wave_base;
    case MPS_PLAN_ARRAY_RB_HOT: *bytes = 0; return nullptr;  // host layouts only
    case MPS_PLAN_ARRAY_RB_HOT_PACKED: *bytes = dp->hot_slots / kPair * 12; return dp->hot;
    case MPS_PLAN_ARRAY_RB_COLD: *bytes = dp->cold ? dp->cold_slots * sizeof(Entry) : 0; return dp->cold;
    case MPS_PLAN_ARRAY_RB_COLD_PACKED: *bytes = dp->cold_packed ? dp->cold_slots / kPair * 12 : 0; return dp->cold_packed;
    case MPS_PLAN_ARRAY_RB_COLD_BEGIN: *bytes = L.cold_begin.size() * sizeof(int); return dp->cold_begin;
    case MPS_PLAN_ARRAY_RB_TABLE_BASE: *bytes = L.table_base.size() * sizeof(int); return dp->table_base;
    case MPS_PLAN_ARRAY_RB_HOT_SRC: *bytes = dp->hot_src ? dp->hot_slots * sizeof(int) : 0; return dp->hot_src;
    case MPS_PLAN_ARRAY_RB_COLD_SRC: *bytes = dp->cold_src ? dp->cold_slots * sizeof(int) : 0; return dp->cold_src;
    default: *bytes = 0; return nullptr;
    }
}
size_t device_bytes_of(const DevicePlan *dp) { return dp->device_bytes; }

}  // namespace mps_rb
