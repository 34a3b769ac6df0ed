// Sweep plans: layout shared by the builder (mpspmm_sweep_host.cpp; its passes
// over the nonzeros also on the device, mpspmm_sweep_build.hip) and the kernel
// (mpspmm_sweep.hip).  Not installed.
//
// The reference walks a partition's nonzeros in row order and gathers the
// dense row of every nonzero from memory (src/MergePathSpMM.cu:426-477); rows
// that straddle partitions are finished with atomics (:445, :477).  Where rows
// are short and X is many times the size of an L2, that order has no locality:
// a gather misses L2 four times in ten.  A sweep plan keeps the arithmetic
// (one fp32 accumulator per output column, a rounded product added per
// nonzero) and changes the order in which the nonzeros are visited:
//
//   * The rows of the matrix are dealt to NP panels, one 1,024-thread
//     workgroup each, so that every panel holds about the same number of
//     nonzeros: largest rows first, each to the panel with the fewest nonzeros
//     so far (rows are dealt in pairs where two of them share a 128-byte line
//     of Y).  A row with more nonzeros than a panel's share is cut into
//     sub-rows that go to different panels; their sums meet in a small
//     fix-up kernel.
//   * A panel keeps one accumulator row per output row in LDS (fp32).  Long
//     rows get several ("pieces": entry k of the row goes to piece k mod P), so
//     that no accumulator row holds more than a fraction of a wavefront's
//     share.  The accumulator rows are dealt to the 16 wavefronts of the
//     workgroup the same way, and belong to that wavefront for the whole
//     kernel: no other wavefront adds to them, so there are no atomics and no
//     barriers for the sums, and every sum has a fixed order.
//   * A wavefront's nonzeros are sorted by column and visited in that order.
//     All wavefronts of all panels start together and hold the same number of
//     nonzeros, so at any time the whole chip gathers from the same narrow
//     range of columns: a row of X is fetched into each L2 about once.  (A
//     workgroup barrier every few rounds keeps the wavefronts of a panel from
//     drifting apart: a SIMD serves its oldest wavefront first.)
//   * An entry is 8 bytes: {column | accumulator row << col_bits, value}.  One
//     instruction handles one entry per lane-group (L lanes x 16 bytes of a row
//     of X: L = 4 for 64-byte rows, 8 for 128-byte column tiles); entries of
//     one instruction never share an accumulator row (the builder moves a
//     second one to the next instruction), so the read-add-write of the
//     accumulators needs no care.  A round is 8 instructions: every lane loads
//     its entry of two windows of 4 with one 16-byte load, and the 4 lanes of
//     a quad pass their entries round with quad permutes.
//   * Rows of X wider than 128 bytes are handled in column tiles of 128 bytes
//     (blockIdx.y): the same stream once per tile.  A row need not fill its last
//     tile (or, below 64 bytes, its only one): lanes past the row's end stay idle.
#ifndef MPSPMM_SWEEP_HPP
#define MPSPMM_SWEEP_HPP

#include <cstdint>
#include <memory>
#include <new>
#include <vector>

namespace mps_sw {

constexpr int kWaves = 16;          // wavefronts of a workgroup
constexpr int kThreads = kWaves * 64;
constexpr int kWin = 4;             // entries of a window: one per lane of a quad
constexpr int kPair = 2;            // windows per lane-group and round: a lane loads its entry of both with one 16-byte load
constexpr int kRoundInstr = kWin * kPair;  // instructions (entries per lane-group) of a round
constexpr int kSyncRounds = 4;      // a workgroup barrier every so many rounds
constexpr int kLdsBytes = 160 * 1024;
constexpr int kMinRowBits = 6;      // an entry word keeps at least this many bits for the accumulator row

// LDS row of accumulator row v: rows that are a multiple of 16 apart (the pieces of one long row that a wavefront
// holds) would otherwise share their banks.  G = accumulator rows per 256 bytes (a power of two).
inline int swizzle(int v, int G) { return v ^ (((v >> 2) ^ (v >> 4) ^ (v >> 6)) & (G - 1)); }

// A vector whose resize() leaves new elements as they are: the stream of a large matrix is hundreds of MB that the
// builder overwrites anyway, and zeroing them first is a serial pass over fresh pages.
template <typename T>
struct LeaveAlone : std::allocator<T> {
    template <typename U>
    struct rebind {
        using other = LeaveAlone<U>;
    };
    template <typename U, typename... Args>
    void construct(U *p, Args &&...args)
    {
        if constexpr (sizeof...(Args) == 0) ::new (static_cast<void *>(p)) U;
        else ::new (static_cast<void *>(p)) U(static_cast<Args &&>(args)...);
    }
};
template <typename T>
using Bulk = std::vector<T, LeaveAlone<T>>;

struct Layout {
    int n = 0, nnz = 0, K = 0, elem_bytes = 4;
    int lanes = 4;        // L: lanes per lane-group; a tile of a row of X is 16 L bytes
    int tiles = 1;        // column tiles per row of X
    int num_panels = 0;   // NP
    int acc_rows = 0;     // accumulator rows per panel in LDS (a multiple of 4); one more holds the sums of the padding
    int col_bits = 0;     // an entry word is column | accumulator row << col_bits
    int piece = 0;        // most entries of a row that one accumulator row takes
    int bank_rows = 1;    // G of swizzle()
    int together = 1;     // instructions whose entries are added up at the same time: 1, or 2 (entry q of windows A and B:
                          // no two entries of such a pair of instructions share an accumulator row)
    long long rounds = 0; // of all wavefronts
    std::vector<int> panel_ptr;     // [NP + 1] a panel's listed rows: rows[panel_ptr[p] .. panel_ptr[p + 1])
    std::vector<int> rows;          // row of Y that a listed row is written to; n + s: partial row s (a sub-row of a split row)
    std::vector<int> piece_ptr;     // [rows + NP] per panel, listed rows + 1 entries: first accumulator row of every listed row
    std::vector<int> wave_meta;     // [NP * 16][2] {first round, rounds} of every wavefront
    std::vector<int> panel_rounds;  // [NP] most rounds of a wavefront of the panel
    Bulk<uint32_t> stream;          // rounds x (64 / L lane-groups) x 4 lanes x {word A, value A, word B, value B}
    Bulk<int> src;                  // original nonzero index of every entry slot (stream order, 2 per 16 bytes), -1 = padding (optional)
    std::vector<int> split_row;     // rows that are cut into sub-rows
    std::vector<int> split_ptr;     // [split rows + 1] their partial rows: split_ptr[i] .. split_ptr[i + 1]
};

struct BuildParams {
    int num_cus = 256;   // panels are made in multiples of this
    int piece = 0;       // 0 = choose
    int acc_rows = 0;    // 0 = what fits in LDS
    int together = 0;    // 0 = choose (2 with 8 lane-groups per wavefront, else 1)
    int elem_bytes = 4;  // of X and Y (values are handed to the builder as fp32 either way)
    bool keep_src = true;
    bool host_build = false;  // create(): the passes over the nonzeros on the host (the device passes build the same layout)
};

constexpr int kNeedHost = -2;  // build_streams_on_device: this layout is for the host passes

// A row as a panel lists it: entries first, first + stride, ... of row `row` of the matrix (a whole row: 0 and 1; sub-row
// j of a row cut into S: j and S), dealt to `pieces` accumulator rows from first_piece on (entry e to piece e mod pieces).
struct ListedRow {
    int row, first, stride, entries, pieces, first_piece;
    long long entries_before;  // of the panel's entries, in listing order
};

// The builder in two parts.  plan_panels: everything that needs row_ptr alone (panels, rows cut across panels, listed
// rows, accumulator rows); it fills the small tables of `out` except wave_meta and panel_rounds.  build_streams: the
// passes over the nonzeros (accumulator rows to wavefronts, entries by column, list scheduling, the stream).
int plan_panels(const int *row_ptr, int n, int nnz, int K, const BuildParams &bp, Layout &out, Bulk<ListedRow> &listed_rows);
int build_streams(const int *row_ptr, const int *col_idx, const float *val, const BuildParams &bp, Layout &out,
                  const Bulk<ListedRow> &listed_rows);

// Host arrays in, layout out.  Returns an mps_status (MPS_ERR_UNSUPPORTED for a row of X that is not a multiple of
// 64 bytes or a matrix whose column ids leave no room for the accumulator row in an entry word).
int build_layout(const int *row_ptr, const int *col_idx, const float *val, int n, int nnz, int K, const BuildParams &bp,
                 Layout &out);

}  // namespace mps_sw
struct mps_plan_info;
namespace mps_sw {
// The sweep_* fields of an mps_plan_info.
void fill_info(const Layout &L, mps_plan_info *info);

#ifdef MPSPMM_DEVICE_HPP
struct DevicePlan;
// build_streams on the device (mpspmm_sweep_build.hip): row_ptr, col_idx and fp32 values on the device in, the stream
// (and the source index of every slot, if bp.keep_src) in device memory out; fills out.wave_meta, out.panel_rounds and
// out.rounds.  Returns an mps_status or kNeedHost; whatever *ds holds afterwards is the caller's to free.
struct DeviceStreams {
    uint32_t *stream = nullptr;
    int *src = nullptr;
    size_t slots = 0, bytes = 0;
};
int build_streams_on_device(const int *d_row_ptr, const int *d_col_idx, const float *d_val, const BuildParams &bp, Layout &out,
                            const Bulk<ListedRow> &listed_rows, hipStream_t st, DeviceStreams *ds);
int create(const int *d_row_ptr, const int *d_col_idx, const void *d_val, int n, int nnz, int K, const BuildParams &bp,
           hipStream_t st, DevicePlan **out);
void destroy(DevicePlan *dp);
int spmm(const DevicePlan *dp, const void *X, void *Y, unsigned phases, hipStream_t st);
int set_values(DevicePlan *dp, const void *d_val, hipStream_t st);
const Layout &layout_of(const DevicePlan *dp);
bool built_on_device(const DevicePlan *dp);  // the passes over the nonzeros ran on the device
size_t device_bytes_of(const DevicePlan *dp);
const void *device_array(const DevicePlan *dp, int which, size_t *bytes);
#endif

}  // namespace mps_sw

#endif
