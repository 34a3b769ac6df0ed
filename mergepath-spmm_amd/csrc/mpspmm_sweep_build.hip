// Sweep plans: the builder's passes over the nonzeros on the device.  The layout is the one that build_streams
// (mpspmm_sweep_host.cpp) makes on the host, entry for entry: the same accumulator rows go to the same wavefronts, a
// wavefront's entries come in the same order (by column, equal columns in listing order), and the list scheduling is
// the same sequential walk - here one thread per wavefront instead of one host thread per panel.
// No counterpart in the reference, whose host side builds the merge-path schedule only (src/MergePathSpMM.cu:300-385).
#include "mpspmm_device.hpp"
#include "mpspmm_hostpar.hpp"
#include "mpspmm_sweep.hpp"

#include <cstring>

#include <rocprim/rocprim.hpp>

#include <algorithm>
#include <vector>

namespace mps_sw {

namespace {

constexpr int kDealThreads = 256;
constexpr int kMaxPieces = 4096;  // accumulator rows of a panel that the deal sorts in LDS (a panel holds at most 2,544)

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

#define SWB_TRY(expr)                                           \
    do {                                                        \
        const hipError_t e_ = (expr);                           \
        if (e_ != hipSuccess) return MPS_ERR_HIP + (int)e_;     \
    } while (0)

// What the device needs of a listed row (ListedRow without what only the host uses)
struct DevRow {
    int row, first, stride, entries, pieces, first_piece;
    unsigned entry_base;  // of the panel's entries, in listing order
    int panel;
};

// One workgroup per panel: the panel's accumulator rows, largest first (equal sizes in index order), each to the
// wavefront with the fewest entries so far (the lowest-numbered one among equals) - deal_largest_first of the host
// builder.  piece_wave: the wavefront of every accumulator row; piece_local: its place among that wavefront's rows;
// wave_entries / wave_pieces: per wavefront.
__global__ __launch_bounds__(kDealThreads) void swb_deal_kernel(const int *__restrict__ panel_ptr, const DevRow *__restrict__ rows,
                                                                 const long long *__restrict__ piece_base,
                                                                 unsigned char *__restrict__ piece_wave,
                                                                 int *__restrict__ piece_local, int *__restrict__ wave_entries,
                                                                 int *__restrict__ wave_pieces, int largest)
{
    __shared__ unsigned key[kMaxPieces];
    __shared__ int size_of[kMaxPieces];
    const int p = blockIdx.x, tid = threadIdx.x;
    const int l0 = panel_ptr[p], l1 = panel_ptr[p + 1];
    const int v = l1 > l0 ? rows[l1 - 1].first_piece + rows[l1 - 1].pieces : 0;
    for (int i = tid; i < kMaxPieces; i += kDealThreads) key[i] = 0xffffffffu;
    __syncthreads();
    for (int l = l0 + tid; l < l1; l += kDealThreads) {
        const DevRow R = rows[l];
        for (int j = 0; j < R.pieces; ++j) {
            const int s = R.entries / R.pieces + (j < R.entries % R.pieces);
            size_of[R.first_piece + j] = s;
            key[R.first_piece + j] = ((unsigned)(largest - s) << 12) | (unsigned)(R.first_piece + j);
        }
    }
    __syncthreads();
    // bitonic sort of the keys (unique: size, then index); the unused places hold the largest key and stay behind
    int N = 2;
    while (N < v) N <<= 1;
    for (int k = 2; k <= N; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = tid; i < N; i += kDealThreads) {
                const int partner = i ^ j;
                if (partner > i) {
                    const unsigned a = key[i], b = key[partner];
                    const bool up = (i & k) == 0;
                    if ((a > b) == up) {
                        key[i] = b;
                        key[partner] = a;
                    }
                }
            }
            __syncthreads();
        }
    if (tid == 0) {
        int load[kWaves], count[kWaves];
        for (int w = 0; w < kWaves; ++w) load[w] = count[w] = 0;
        const long long base = piece_base[p];
        for (int k = 0; k < v; ++k) {
            const int i = (int)(key[k] & 0xfffu);
            int best = 0;
            for (int w = 1; w < kWaves; ++w)
                if (load[w] < load[best]) best = w;
            piece_wave[base + i] = (unsigned char)best;
            piece_local[base + i] = count[best]++;
            load[best] += size_of[i];
        }
        for (int w = 0; w < kWaves; ++w) {
            wave_entries[p * kWaves + w] = load[w];
            wave_pieces[p * kWaves + w] = count[w];
        }
    }
}

// Every entry of the matrix to the segment of its (panel, wavefront), in any order: key = column, then its place in
// the panel's listing (which makes the order after the sort the host builder's); value = accumulator row and nonzero.
constexpr int kPerThread = 8;
__global__ __launch_bounds__(256) void swb_scatter_kernel(const int *__restrict__ rp, const int *__restrict__ ci,
                                                           const DevRow *__restrict__ rows, const long long *__restrict__ row_first,
                                                           int listed, long long entries, const long long *__restrict__ piece_base,
                                                           const unsigned char *__restrict__ piece_wave,
                                                           const unsigned *__restrict__ seg_begin, unsigned *__restrict__ seg_cursor,
                                                           unsigned long long *__restrict__ keys, unsigned long long *__restrict__ values)
{
    const long long g0 = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * kPerThread;
    if (g0 >= entries) return;
    // the listed row of entry g0: the last one that starts at or before it (row_first has listed + 1 entries)
    int lo = 0, hi = listed;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (row_first[mid] <= g0) lo = mid; else hi = mid;
    }
    int l = lo;
    const int count = (int)min((long long)kPerThread, entries - g0);
    int seg_of[kPerThread];
    unsigned long long key_of[kPerThread], value_of[kPerThread];
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
        seg_of[i] = -1;
        if (i >= count) continue;
        const long long g = g0 + i;
        while (row_first[l + 1] <= g) ++l;  // (rows without entries are stepped over)
        const DevRow R = rows[l];
        const int e = (int)(g - row_first[l]);
        const long long at = (long long)rp[R.row] + R.first + (long long)e * R.stride;
        const int vl = R.first_piece + e % R.pieces;
        seg_of[i] = R.panel * kWaves + piece_wave[piece_base[R.panel] + vl];
        key_of[i] = ((unsigned long long)(unsigned)ci[at] << 32) | (unsigned long long)(R.entry_base + (unsigned)e);
        value_of[i] = ((unsigned long long)(unsigned)vl << 32) | (unsigned long long)(unsigned)at;
    }
    // neighbours that go to the same segment (the entries of a long row) take their places with one atomic
    unsigned pos = 0;
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
        if (seg_of[i] < 0) continue;
        if (i == 0 || seg_of[i] != seg_of[i - 1]) {
            unsigned run = 1;
#pragma unroll
            for (int j = i + 1; j < kPerThread; ++j) {
                if (seg_of[j] != seg_of[i]) break;
                ++run;
            }
            pos = seg_begin[seg_of[i]] + atomicAdd(&seg_cursor[seg_of[i]], run);
        }
        keys[pos] = key_of[i];
        values[pos] = value_of[i];
        ++pos;
    }
}

// One thread per wavefront of the layout: its entries, by column, each to the first group (an instruction, or a pair
// of instructions) from the frontier on that has room and does not yet hold an entry of the same accumulator row -
// the loop of build_streams.  slot: group * group_slots + place; rounds: per wavefront.
__global__ __launch_bounds__(64) void swb_schedule_kernel(const unsigned long long *__restrict__ values,
                                                           const unsigned *__restrict__ seg_begin, int segments,
                                                           const long long *__restrict__ piece_base,
                                                           const int *__restrict__ piece_local,
                                                           const long long *__restrict__ wave_piece_base, int *__restrict__ last,
                                                           unsigned char *__restrict__ fill, unsigned *__restrict__ slot,
                                                           int *__restrict__ rounds, int group_slots, int groups_per_round)
{
    const int seg = blockIdx.x * blockDim.x + threadIdx.x;
    if (seg >= segments) return;
    const unsigned e0 = seg_begin[seg], e1 = seg_begin[seg + 1];
    const long long pieces0 = piece_base[seg / kWaves];
    int *my_last = last + wave_piece_base[seg];                    // [pieces of the wavefront], -1 at the start
    unsigned char *my_fill = fill + (size_t)e0 + 2 * (size_t)seg;  // [entries + 2], 0 at the start
    long long frontier = 0, top = 0;
    for (unsigned e = e0; e < e1; ++e) {
        const int vl = (int)(values[e] >> 32);
        int *lastp = my_last + piece_local[pieces0 + vl];
        long long t = max(frontier, (long long)*lastp + 1);
        while (my_fill[t] >= group_slots) ++t;
        slot[e] = (unsigned)(t * group_slots + my_fill[t]);
        ++my_fill[t];
        *lastp = (int)t;
        top = max(top, t + 1);
        while (my_fill[frontier] == group_slots) ++frontier;
    }
    rounds[seg] = (int)((top + groups_per_round - 1) / groups_per_round);
}

// The stream before the entries: every slot holds the padding (column 0, value 0, the spare accumulator row).
__global__ __launch_bounds__(256) void swb_pad_kernel(uint2 *__restrict__ stream, size_t slots, unsigned pad_word)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < slots) stream[i] = make_uint2(pad_word, 0u);
}

// Every entry to its slot of the stream (the index arithmetic of build_streams).
__global__ __launch_bounds__(256) void swb_emit_kernel(const unsigned long long *__restrict__ keys,
                                                        const unsigned long long *__restrict__ values,
                                                        const unsigned *__restrict__ slot, const unsigned *__restrict__ seg_begin,
                                                        int segments, const int *__restrict__ wave_meta,
                                                        const float *__restrict__ val, uint32_t *__restrict__ stream,
                                                        int *__restrict__ src, unsigned entries, int gpw, int together, int G,
                                                        int col_bits)
{
    const unsigned e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= entries) return;
    int lo = 0, hi = segments;  // the segment of entry e: seg_begin[seg] <= e < seg_begin[seg + 1]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (seg_begin[mid] <= e) lo = mid; else hi = mid;
    }
    const int group_slots = gpw * together, groups_per_round = kRoundInstr / together, words_per_round = gpw * kWin * 4;
    const unsigned s = slot[e];
    const long long t = s / (unsigned)group_slots, i = s % (unsigned)group_slots;
    const long long round = t / groups_per_round, g = i % gpw;
    const long long w2 = together == 2 ? i / gpw : (t % kRoundInstr) / kWin, q = t % kWin;
    const size_t at = (size_t)wave_meta[2 * lo] * (size_t)words_per_round +
                      (size_t)((round * gpw * kWin + g * kWin + q) * 4 + w2 * 2);
    const unsigned col = (unsigned)(keys[e] >> 32);
    const int vl = (int)(values[e] >> 32), nz = (int)(unsigned)values[e];
    const int place = vl ^ (((vl >> 2) ^ (vl >> 4) ^ (vl >> 6)) & (G - 1));  // mps_sw::swizzle
    stream[at] = col | ((unsigned)place << col_bits);
    stream[at + 1] = __float_as_uint(val[nz]);
    if (src) src[at / 2] = nz;
}

}  // namespace

int build_streams_on_device(const int *d_rp, const int *d_ci, const float *d_val, const BuildParams &bp, Layout &out,
                            const Bulk<ListedRow> &listed_rows, hipStream_t st, DeviceStreams *ds)
{
    const int NP = out.num_panels, L = out.lanes, gpw = 64 / L, together = out.together;
    const int group_slots = gpw * together, groups_per_round = kRoundInstr / together, words_per_round = gpw * kWin * 4;
    const int listed = (int)listed_rows.size(), segments = NP * kWaves;
    const long long entries = out.nnz;
    if (out.acc_rows > kMaxPieces || out.piece >= (1 << 20) || entries >= (1ll << 31)) return kNeedHost;

    // the listed rows as the kernels read them; where the entries of every listed row and the accumulator rows of every
    // panel start
    std::vector<DevRow> rows((size_t)listed);
    std::vector<long long> row_first((size_t)listed + 1, 0), piece_base((size_t)NP + 1, 0), panel_first((size_t)NP + 1, 0);
    for (int p = 0; p < NP; ++p) {
        const int l0 = out.panel_ptr[(size_t)p], l1 = out.panel_ptr[(size_t)p + 1];
        long long in_panel = 0;
        int pieces = 0;
        if (l1 > l0) {
            const ListedRow &R = listed_rows[(size_t)l1 - 1];
            in_panel = R.entries_before + R.entries;
            pieces = R.first_piece + R.pieces;
        }
        if (in_panel >= (1ll << 32)) return kNeedHost;
        panel_first[(size_t)p + 1] = panel_first[(size_t)p] + in_panel;
        piece_base[(size_t)p + 1] = piece_base[(size_t)p] + pieces;
    }
    mps_host::parallel_for(NP, 16, [&](int64_t lo, int64_t hi) {
        for (int64_t p = lo; p < hi; ++p)
            for (int l = out.panel_ptr[(size_t)p]; l < out.panel_ptr[(size_t)p + 1]; ++l) {
                const ListedRow &R = listed_rows[(size_t)l];
                rows[(size_t)l] = DevRow{R.row, R.first, R.stride, R.entries, R.pieces, R.first_piece, (unsigned)R.entries_before, (int)p};
                row_first[(size_t)l] = panel_first[(size_t)p] + R.entries_before;
            }
    });
    row_first[(size_t)listed] = panel_first[(size_t)NP];
    if (row_first[(size_t)listed] != entries) return MPS_ERR_INVALID_CSR;
    const long long pieces_all = piece_base[(size_t)NP];

    Scratch d_rows, d_row_first, d_piece_base, d_panel_ptr, d_piece_wave, d_piece_local, d_wave_entries, d_wave_pieces;
    SWB_TRY(d_rows.get(rows.size() * sizeof(DevRow)));
    SWB_TRY(d_row_first.get(row_first.size() * sizeof(long long)));
    SWB_TRY(d_piece_base.get(piece_base.size() * sizeof(long long)));
    SWB_TRY(d_panel_ptr.get(out.panel_ptr.size() * sizeof(int)));
    SWB_TRY(d_piece_wave.get((size_t)pieces_all));
    SWB_TRY(d_piece_local.get((size_t)pieces_all * sizeof(int)));
    SWB_TRY(d_wave_entries.get((size_t)segments * sizeof(int)));
    SWB_TRY(d_wave_pieces.get((size_t)segments * sizeof(int)));
    SWB_TRY(hipMemcpyAsync(d_rows.p, rows.data(), rows.size() * sizeof(DevRow), hipMemcpyHostToDevice, st));
    SWB_TRY(hipMemcpyAsync(d_row_first.p, row_first.data(), row_first.size() * sizeof(long long), hipMemcpyHostToDevice, st));
    SWB_TRY(hipMemcpyAsync(d_piece_base.p, piece_base.data(), piece_base.size() * sizeof(long long), hipMemcpyHostToDevice, st));
    SWB_TRY(hipMemcpyAsync(d_panel_ptr.p, out.panel_ptr.data(), out.panel_ptr.size() * sizeof(int), hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(swb_deal_kernel, dim3((unsigned)NP), dim3(kDealThreads), 0, st, d_panel_ptr.as<int>(), d_rows.as<DevRow>(),
                       d_piece_base.as<long long>(), d_piece_wave.as<unsigned char>(), d_piece_local.as<int>(),
                       d_wave_entries.as<int>(), d_wave_pieces.as<int>(), std::max(out.piece, 1));
    std::vector<int> wave_entries((size_t)segments), wave_pieces((size_t)segments);
    SWB_TRY(hipMemcpyAsync(wave_entries.data(), d_wave_entries.p, (size_t)segments * sizeof(int), hipMemcpyDeviceToHost, st));
    SWB_TRY(hipMemcpyAsync(wave_pieces.data(), d_wave_pieces.p, (size_t)segments * sizeof(int), hipMemcpyDeviceToHost, st));
    SWB_TRY(hipStreamSynchronize(st));
    std::vector<unsigned> seg_begin((size_t)segments + 1, 0u);
    std::vector<long long> wave_piece_base((size_t)segments + 1, 0);
    for (int s = 0; s < segments; ++s) {
        seg_begin[(size_t)s + 1] = seg_begin[(size_t)s] + (unsigned)wave_entries[(size_t)s];
        wave_piece_base[(size_t)s + 1] = wave_piece_base[(size_t)s] + wave_pieces[(size_t)s];
    }
    if ((long long)seg_begin[(size_t)segments] != entries) return MPS_ERR_INVALID_CSR;

    // entries to their segments, sorted there by (column, place in the listing)
    Scratch d_seg_begin, d_seg_cursor, d_keys, d_keys2, d_values, d_values2, d_temp;
    const size_t ne = (size_t)entries;
    SWB_TRY(d_seg_begin.get(seg_begin.size() * sizeof(unsigned)));
    SWB_TRY(d_seg_cursor.get((size_t)segments * sizeof(unsigned)));
    SWB_TRY(d_keys.get(ne * sizeof(unsigned long long)));
    SWB_TRY(d_keys2.get(ne * sizeof(unsigned long long)));
    SWB_TRY(d_values.get(ne * sizeof(unsigned long long)));
    SWB_TRY(d_values2.get(ne * sizeof(unsigned long long)));
    SWB_TRY(hipMemcpyAsync(d_seg_begin.p, seg_begin.data(), seg_begin.size() * sizeof(unsigned), hipMemcpyHostToDevice, st));
    SWB_TRY(hipMemsetAsync(d_seg_cursor.p, 0, (size_t)segments * sizeof(unsigned), st));
    if (entries > 0) {
        const long long threads = (entries + kPerThread - 1) / kPerThread;
        hipLaunchKernelGGL(swb_scatter_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, d_rp, d_ci,
                           d_rows.as<DevRow>(), d_row_first.as<long long>(), listed, entries, d_piece_base.as<long long>(),
                           d_piece_wave.as<unsigned char>(), d_seg_begin.as<unsigned>(), d_seg_cursor.as<unsigned>(),
                           d_keys.as<unsigned long long>(), d_values.as<unsigned long long>());
        SWB_TRY(hipGetLastError());
        size_t temp_bytes = 0;
        const unsigned end_bit = 32u + (unsigned)out.col_bits;
        SWB_TRY(rocprim::segmented_radix_sort_pairs(nullptr, temp_bytes, d_keys.as<unsigned long long>(),
                                                    d_keys2.as<unsigned long long>(), d_values.as<unsigned long long>(),
                                                    d_values2.as<unsigned long long>(), (unsigned)entries, (unsigned)segments,
                                                    d_seg_begin.as<unsigned>(), d_seg_begin.as<unsigned>() + 1, 0u, end_bit, st));
        SWB_TRY(d_temp.get(temp_bytes));
        SWB_TRY(rocprim::segmented_radix_sort_pairs(d_temp.p, temp_bytes, d_keys.as<unsigned long long>(),
                                                    d_keys2.as<unsigned long long>(), d_values.as<unsigned long long>(),
                                                    d_values2.as<unsigned long long>(), (unsigned)entries, (unsigned)segments,
                                                    d_seg_begin.as<unsigned>(), d_seg_begin.as<unsigned>() + 1, 0u, end_bit, st));
    }

    // list scheduling, one thread per wavefront
    Scratch d_wave_piece_base, d_last, d_fill, d_slot, d_rounds;
    SWB_TRY(d_wave_piece_base.get(wave_piece_base.size() * sizeof(long long)));
    SWB_TRY(d_last.get((size_t)pieces_all * sizeof(int)));
    SWB_TRY(d_fill.get(ne + 2 * (size_t)segments + 2));
    SWB_TRY(d_slot.get(ne * sizeof(unsigned)));
    SWB_TRY(d_rounds.get((size_t)segments * sizeof(int)));
    SWB_TRY(hipMemcpyAsync(d_wave_piece_base.p, wave_piece_base.data(), wave_piece_base.size() * sizeof(long long),
                           hipMemcpyHostToDevice, st));
    SWB_TRY(hipMemsetAsync(d_last.p, 0xff, (size_t)pieces_all * sizeof(int), st));
    SWB_TRY(hipMemsetAsync(d_fill.p, 0, ne + 2 * (size_t)segments + 2, st));
    hipLaunchKernelGGL(swb_schedule_kernel, dim3((unsigned)((segments + 63) / 64)), dim3(64), 0, st,
                       d_values2.as<unsigned long long>(), d_seg_begin.as<unsigned>(), segments, d_piece_base.as<long long>(),
                       d_piece_local.as<int>(), d_wave_piece_base.as<long long>(), d_last.as<int>(), d_fill.as<unsigned char>(),
                       d_slot.as<unsigned>(), d_rounds.as<int>(), group_slots, groups_per_round);
    std::vector<int> rounds((size_t)segments);
    SWB_TRY(hipMemcpyAsync(rounds.data(), d_rounds.p, (size_t)segments * sizeof(int), hipMemcpyDeviceToHost, st));
    SWB_TRY(hipStreamSynchronize(st));

    // where every wavefront's rounds start
    out.wave_meta.assign((size_t)segments * 2, 0);
    out.panel_rounds.assign((size_t)NP, 0);
    long long first_round = 0;
    for (int p = 0; p < NP; ++p) {
        int most = 0;
        for (int w = 0; w < kWaves; ++w) {
            const int r = rounds[(size_t)p * kWaves + w];
            out.wave_meta[((size_t)p * kWaves + w) * 2] = (int)first_round;
            out.wave_meta[((size_t)p * kWaves + w) * 2 + 1] = r;
            first_round += r;
            most = std::max(most, r);
        }
        out.panel_rounds[(size_t)p] = most;
    }
    out.rounds = first_round;
    if (out.rounds * (long long)words_per_round / 4 > 0x7fffffffll) return MPS_ERR_UNSUPPORTED;  // 16-byte units index the stream

    // the stream
    Scratch d_wave_meta;
    const size_t words = (size_t)out.rounds * (size_t)words_per_round;
    SWB_TRY(d_wave_meta.get(out.wave_meta.size() * sizeof(int)));
    SWB_TRY(hipMemcpyAsync(d_wave_meta.p, out.wave_meta.data(), out.wave_meta.size() * sizeof(int), hipMemcpyHostToDevice, st));
    SWB_TRY(hipMalloc(reinterpret_cast<void **>(&ds->stream), (words ? words : 1) * sizeof(uint32_t)));
    ds->bytes += (words ? words : 1) * sizeof(uint32_t);
    ds->slots = words / 2;
    if (bp.keep_src) {
        SWB_TRY(hipMalloc(reinterpret_cast<void **>(&ds->src), (ds->slots ? ds->slots : 1) * sizeof(int)));
        ds->bytes += (ds->slots ? ds->slots : 1) * sizeof(int);
        SWB_TRY(hipMemsetAsync(ds->src, 0xff, ds->slots * sizeof(int), st));
    }
    if (ds->slots > 0)
        hipLaunchKernelGGL(swb_pad_kernel, dim3((unsigned)((ds->slots + 255) / 256)), dim3(256), 0, st,
                           reinterpret_cast<uint2 *>(ds->stream), ds->slots, (unsigned)out.acc_rows << out.col_bits);
    if (entries > 0)
        hipLaunchKernelGGL(swb_emit_kernel, dim3((unsigned)((entries + 255) / 256)), dim3(256), 0, st,
                           d_keys2.as<unsigned long long>(), d_values2.as<unsigned long long>(), d_slot.as<unsigned>(),
                           d_seg_begin.as<unsigned>(), segments, d_wave_meta.as<int>(), d_val, ds->stream, ds->src,
                           (unsigned)entries, gpw, together, out.bank_rows, out.col_bits);
    SWB_TRY(hipGetLastError());
    SWB_TRY(hipStreamSynchronize(st));
    return MPS_OK;
}

}  // namespace mps_sw
