// Row-block plans: layout shared by the host-side builder
// (mpspmm_rowblock_host.cpp) and the device side (mpspmm_rowblock.hip).
// Not installed.
//
// The reference walks every merge-path partition with one accumulator per
// output column and gathers the dense row of every nonzero from memory
// (src/MergePathSpMM.cu:426-477).  On MI355X that gather is what limits a
// matrix with long rows: a 64-byte row of X is one L1->L2 request however it
// is scheduled.  A row-block plan keeps the arithmetic and changes where the
// operands live:
//
//   * The rows of the matrix are cut into NB contiguous blocks of about equal
//     nonzero count, one per 1,024-thread workgroup (one workgroup per CU).
//     A block's output rows are accumulated in LDS (fp32) and written to Y
//     once: no partial rows in memory, no carry-out records, no second kernel.
//   * The columns are dealt to T steps.  The T * H columns with the most
//     nonzeros are "hot": step t keeps the rows of X of its H hot columns in
//     an LDS table, and their nonzeros gather from there.  The other columns
//     are "cold": step t owns a contiguous range of column ids (equal cold
//     nonzero counts per step), gathered through L2, so that the CUs of an
//     XCD, which walk the steps at about the same pace, share a few hundred
//     KiB of X at a time.
//   * Within (block, step) the nonzeros are grouped into windows of 4 entries
//     of one row (a row's last hot window and last cold window of the step
//     are padded: value 0, the last index repeated).  The windows in row order
//     (a row's hot ones, then its cold ones) are cut into 16 runs of about
//     equal length (see kCutSlack), one per wavefront; a wavefront's hot windows are then dealt evenly and in
//     order to its 16 lane-groups, and so are its cold ones.  Every lane-group
//     therefore walks two short streams (hot: LDS gathers, cold: L2 gathers)
//     of the same length as its neighbours': no divergence.  A round of a
//     stream holds two windows per lane-group, side by side, so that a lane
//     reads its entry of both with one 16-byte load.
//   * An entry is 8 bytes: {index | rows_advanced << index_bits, value}.
//     index is the LDS table slot (hot) or the column id (cold);
//     rows_advanced, in a window's first entry only, is how many block-local
//     rows lie between this window and the previous one of the same
//     lane-group stream (for the first one: between it and the first row of
//     the wavefront's run).
//   * When the row changes, a lane-group adds its partial sums to the row's
//     LDS accumulator (plain read-add-write).  That is safe because a row is
//     added to directly only by the lane-group in whose stream it ends.  The
//     sums a lane-group holds at the end of its run (its last row may go on
//     in the next group's stream) are combined after the walk, in lane-group
//     order, by the first lane-group of every stretch of equal rows.  Only
//     the first row of a wavefront's run can be shared with another
//     wavefront: its sums go to a per-wavefront slot, and the slots are added
//     by one wavefront, in wavefront order, after the step's barrier.
//     Results do not depend on timing.
#ifndef MPSPMM_ROWBLOCK_HPP
#define MPSPMM_ROWBLOCK_HPP

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <functional>
#include <new>
#include <vector>

namespace mps_rb {

constexpr int kWaves = 16;         // wavefronts of a workgroup, each walks nonzeros
constexpr int kWaveSlots = 16;     // stride of the per-wavefront tables
constexpr int kGroups = 16;        // lane-groups per wavefront (4 lanes x 4 columns, K = 16 fp32)
constexpr int kWin = 4;            // entries of a window: one per lane of a lane-group
constexpr int kPair = 2;           // windows of a lane-group per round: a lane loads its entry of both with one 16-byte load
constexpr int kRoundEntries = kGroups * kWin * kPair;  // 128 entries = 1 KiB per round
constexpr int kLdsBytes = 160 * 1024;
// shared-row slots [16][16] floats, their rows [16]
constexpr int kSlotBytes = kWaveSlots * 16 * 4 + kWaveSlots * 4;
constexpr int kMaxTableRows = 1536;  // six 16-byte pieces per thread when a table is moved

struct Entry {
    uint32_t word;  // index | rows_advanced << index_bits
    float val;
};

// Packed hot stream, what the device reads: the table slot of a hot entry needs 11 bits (kMaxTableRows <= 2048) and a
// window advances fewer than 1,024 rows (a block holds at most 1,024), so a lane's share of a round shrinks from 16
// to 12 bytes:
//   {value A, value B, half A | half B << 16},  half = slot | piece << kPackedSlotBits,
// where the 5-bit pieces of a window's entries 0 and 1 are the low and the high half of its rows_advanced (entries
// 2 and 3 carry 0).  A round is then 64 x 12 = 768 bytes; rounds and lanes keep their order.
constexpr int kPackedSlotBits = 11;
constexpr int kPackedPieceBits = 5;
constexpr uint32_t kPackedAdvMax = (1u << (2 * kPackedPieceBits)) - 1u;
constexpr int kPackedRoundWords = 64 * 3;

// A vector whose resize() hands out zeroed memory without writing to it: large blocks come from the system as
// untouched zero pages, which the builder's threads then touch as they fill them, instead of one thread writing
// zeros over tens of megabytes first.  (An Entry of zero bytes is {word 0, value 0.f}: the padding.)
template <typename T>
struct ZeroPages {
    using value_type = T;
    template <typename U>
    struct rebind {
        using other = ZeroPages<U>;
    };
    ZeroPages() = default;
    template <typename U>
    ZeroPages(const ZeroPages<U> &) {}
    T *allocate(size_t count)
    {
        void *p = std::calloc(count ? count : 1, sizeof(T));
        if (!p) throw std::bad_alloc();
        return static_cast<T *>(p);
    }
    void deallocate(T *p, size_t) { std::free(p); }
    template <typename U, typename... Args>
    void construct(U *p, Args &&...args)
    {
        if constexpr (sizeof...(Args) > 0) ::new (static_cast<void *>(p)) U(static_cast<Args &&>(args)...);
    }
    template <typename U>
    bool operator==(const ZeroPages<U> &) const { return true; }
    template <typename U>
    bool operator!=(const ZeroPages<U> &) const { return false; }
};
template <typename T>
using Zeroed = std::vector<T, ZeroPages<T>>;

struct Layout {
    int n = 0, nnz = 0, K = 16;
    int steps = 0;        // T
    int table_rows = 0;   // H
    int acc_rows = 0;     // rows of LDS accumulators per workgroup (>= rows of every block)
    int num_blocks = 0;   // NB
    int hot_bits = 0, cold_bits = 0;
    long long hot_nnz = 0;
    long long hot_rounds = 0, cold_rounds = 0;
    std::vector<int> block_row;         // [NB + 1]
    std::vector<int> hot_cols;          // [T][H] column of every table slot, -1 = unused
    std::vector<int> cold_begin;        // [T + 1] column-id range of every step's cold columns
    std::vector<int> table_base;        // [NB] local tables: block b's table of step t is X[base[b] + t H .. base[b] + (t + 1) H); else empty
    std::vector<int> table_used;        // [NB] local tables: rows of the block's last table that its entries refer to (the rest is not loaded)
    std::vector<int> meta;              // [NB][T][16][4] {hot entries, cold entries, first local row, 0}; [..][15] unused
    std::vector<long long> wave_base;   // [NB * 16][2] first round of the wavefront's hot / cold stream; [..][15]: where the block's streams end
    Zeroed<Entry> hot, cold;            // rounds of 64 entries
    std::vector<int> hot_src, cold_src; // original nonzero index per entry slot, -1 = padding (optional)
    Zeroed<uint32_t> hot_packed;        // the hot stream in packed form
    Zeroed<uint32_t> cold_packed;       // the cold stream in packed form; empty if it does not fit (see pack_cold_stream)
    int cold_index_bits = 0;            // of a packed cold entry's 16 bits, those of the column (counted from cold_begin[t])
};

struct BuildParams {
    int steps = 0;       // 0 = choose
    int table_rows = 0;  // 0 = what fits in LDS beside the accumulators
    int block_rows = 0;  // 0 = choose; otherwise the most rows a block may hold
    int num_cus = 256;
    bool keep_src = true;
    // build_layout gives up (kNotWorthwhile) ...
    double max_local_share = 1.0;             // when the blocks find a larger share of the nonzeros in column ranges of their own
    double max_longest_row = 0.0;             // when the longest row has more than this many times nnz / num_cus nonzeros (0: never)
    double min_table_share_short_rows = 0.0;  // when rows are many and short and the first table serves a smaller share of the nonzeros
    double min_local_cover = 0.6;             // when the columns are local (max_local_share) and local tables would serve a smaller share
    bool local_tables = false;                // local tables whatever the matrix looks like
    bool host_build = false;                  // create(): every pass over the nonzeros on the host (the device passes build the same layout)
};

constexpr int kNotWorthwhile = -1;  // build_layout: one of the three limits of BuildParams not met
constexpr int kNeedHost = -2;       // plan_columns: the layout asks for the column indices on the host (local tables)

// Where a column's nonzeros go: the step, and the slot of the step's LDS table (-1: cold, gathered through L2).
struct ColumnMap {
    std::vector<int16_t> step;  // per column
    std::vector<int16_t> slot;  // per column: table slot, -1 = cold
    // local tables: block b's table of step t holds the columns base[b] + t H .. base[b] + (t + 1) H - 1; the columns
    // outside base[b] .. base[b] + T H - 1 are cold, in the first step (below) or the last (above)
    const int *base = nullptr;
    int H = 0, T = 1;
    int step_of(int b, int c) const
    {
        if (!base) return step[(size_t)c];
        const long long d = (long long)c - base[b];
        return d < 0 ? 0 : (int)std::min<long long>(d / H, T - 1);
    }
    int slot_of(int b, int c) const
    {
        if (!base) return slot[(size_t)c];
        const long long d = (long long)c - base[b];
        return d >= 0 && d < (long long)T * H ? (int)(d % H) : -1;
    }
};

// The builder in its parts, so that the passes over the nonzeros can run where the nonzeros are.
// plan_blocks: the row blocks, the accumulator rows and the most table rows that fit beside them (from row_ptr alone).
int plan_blocks(const int *row_ptr, int n, int nnz, const BuildParams &bp, Layout &out, int *table_rows);
// plan_columns: steps, tables, hot and cold columns.  deg[c]: nonzeros of column c.  block_ranges(R, own, busiest):
// *own = over all blocks, the nonzeros in the block's busiest of R equal column ranges; *busiest = the nonzeros of the
// busiest range of the whole matrix.  col_idx may be null: then kNeedHost comes back where the layout needs it
// (local tables).  Other returns: an mps_status, or kNotWorthwhile.
int plan_columns(const int *row_ptr, const int *col_idx, int n, int nnz, const BuildParams &bp, Layout &out, int table_rows,
                 const int *deg, const std::function<void(int, long long *, long long *)> &block_ranges, ColumnMap &cm);
#if defined(__HIP__) || defined(__HIPCC__)
#define MPS_RB_HD __host__ __device__
#else
#define MPS_RB_HD
#endif
// i-th element of a list of len entries dealt evenly and in order to 16 lane-groups (the first len % 16 groups hold one
// entry more): its lane-group g and its place j there.
MPS_RB_HD inline void deal(int len, int i, int *g, int *j)
{
    const int base = len / kGroups, rem = len % kGroups, big = base + 1;
    if (i < rem * big) {
        *g = i / big;
        *j = i - *g * big;
    } else {
        const int i2 = i - rem * big;
        *g = rem + i2 / base;
        *j = i2 % base;
    }
}
// bits that hold the values 0..v
inline int bits_for(long long v)
{
    int b = 1;
    while ((v >> b) != 0) ++b;
    return b;
}
// rounds (two windows per lane-group each) that a wavefront needs for `windows` windows dealt to its 16 lane-groups
MPS_RB_HD inline int rounds_for(int windows) { return (windows / kGroups + (windows % kGroups != 0) + kPair - 1) / kPair; }

// Where the runs of a step are cut.  A step's E windows, in row order (a row's hot windows, then its cold ones), go
// to the 16 wavefronts in runs of about E / 16; a run's hot and cold windows fill rounds of 32, and the last round of
// either kind is walked and read like a full one however few windows it holds.  So run w begins not at w E / 16 but
// at the window within kCutSlack of it (a fraction of a run's length, either side) that leaves the least padding in
// the rounds of run w - 1; among equals the nearest to w E / 16, then the first.  (232,965-row power-law matrix, 16
// steps: 6.5 % of the entry slots were padding of last rounds and 96 % of the runs had a partly filled round of
// either kind with the cuts at w E / 16; 1.7 % and half of the runs with these.)  A step of fewer than 16 x
// kCutSlack windows is cut at w E / 16.
constexpr int kCutSlack = 8;  // the slack is 1 / kCutSlack of a run
MPS_RB_HD inline int round_padding(int windows) { return rounds_for(windows) * (kGroups * kPair) - windows; }
// what decides between two places for a cut: padding, then distance from the equal cut, then the place itself
MPS_RB_HD inline unsigned long long cut_key(int hot_in_run, int cold_in_run, long long place, long long equal_cut)
{
    const long long away = place < equal_cut ? equal_cut - place : place - equal_cut;
    return ((unsigned long long)(round_padding(hot_in_run) + round_padding(cold_in_run)) << 56) |
           ((unsigned long long)away << 32) | (unsigned long long)place;
}

// Host arrays in, layout out.  Returns an mps_status.
int build_layout(const int *row_ptr, const int *col_idx, const float *val, int n, int nnz, int K,
                 const BuildParams &bp, Layout &out);

// Fills out.hot_packed from out.hot; false if the packed form cannot hold it (no layout of build_layout does that).
bool pack_hot_stream(Layout &out);

// Fills out.cold_packed from out.cold, 12 bytes per lane and round like the hot stream: {value A, value B, half A |
// half B << 16}.  A half holds the column minus the first column of the step's range in its low cold_index_bits
// (12 to 15, what the widest range needs) and, above them, a piece of the window's rows_advanced: entry e of a window
// carries bits [e * p, (e + 1) * p) of it, p = 16 - cold_index_bits.  Returns false and leaves cold_packed empty when
// a range is wider than 32,768 columns or a window advances more rows than 4 p bits hold: the kernel then reads
// out.cold as it is.
bool pack_cold_stream(Layout &out);

// Steps the library picks for a matrix when the caller names none.
int default_steps(int n, long long nnz, int table_rows, int num_blocks, const long long *table_nnz, int tables);

#ifdef MPSPMM_DEVICE_HPP
// Device side (mpspmm_rowblock.hip), for translation units that include the HIP runtime.
struct DevicePlan;
int create(const int *d_row_ptr, const int *d_col_idx, const float *d_val, int n, int nnz, int K, const BuildParams &bp,
           hipStream_t st, DevicePlan **out);
void destroy(DevicePlan *dp);
int spmm(const DevicePlan *dp, const float *X, float *Y, unsigned phases, hipStream_t st);
int set_values(DevicePlan *dp, const float *d_val, hipStream_t st);
const Layout &layout_of(const DevicePlan *dp);
bool built_on_device(const DevicePlan *dp);  // the passes over the nonzeros ran on the device
size_t device_bytes_of(const DevicePlan *dp);
// Device array `which` (MPS_PLAN_ARRAY_RB_*) and its size in bytes; nullptr if the plan does not hold it.
const void *device_array(const DevicePlan *dp, int which, size_t *bytes);
#endif

}  // namespace mps_rb

#endif
