// Sweep plans, host side: the layout builder (see mpspmm_sweep.hpp) and its
// C entry points.  No counterpart in the reference, whose host side builds
// the merge-path schedule only (src/MergePathSpMM.cu:300-385).
#include "mpspmm.h"
#include "mpspmm_hostpar.hpp"
#include "mpspmm_sweep.hpp"

#include <algorithm>
#include <atomic>
#include <cstring>
#include <new>
#include <numeric>
#include <queue>

namespace mps_sw {

namespace {

struct Item {          // what is dealt to panels: a row, a pair of rows, or a sub-row of a split row
    long long nnz;
    int pieces;        // accumulator rows it needs
    int row;           // first row
    int nrows;         // 1 or 2
    int sub;           // -1, or the sub-row index of a split row
};

struct Entry {
    int col;
    int vloc;          // accumulator row, panel-local
    float val;
    int src;
};

int bits_for(unsigned v)
{
    int b = 0;
    while (v) {
        ++b;
        v >>= 1;
    }
    return b < 1 ? 1 : b;
}

// Entries by column, equal columns in the order they came (a radix sort from the low digits up: a wavefront's entries
// are a few thousand 16-byte records, and a comparison sort of them was half of the builder's time).
void sort_by_column(std::vector<Entry> &E, std::vector<Entry> &tmp, std::vector<int> &count, int col_bits)
{
    if (E.size() < 64) {
        std::stable_sort(E.begin(), E.end(), [](const Entry &a, const Entry &b) { return a.col < b.col; });
        return;
    }
    const int passes = (col_bits + 10) / 11, digit_bits = (col_bits + passes - 1) / passes;
    const uint32_t mask = (1u << digit_bits) - 1u;
    tmp.resize(E.size());
    Entry *from = E.data(), *to = tmp.data();
    for (int p = 0; p < passes; ++p) {
        const int shift = p * digit_bits;
        count.assign((size_t)mask + 2, 0);
        for (size_t i = 0; i < E.size(); ++i) ++count[(((uint32_t)from[i].col >> shift) & mask) + 1];
        for (size_t d = 0; d <= mask; ++d) count[d + 1] += count[d];
        for (size_t i = 0; i < E.size(); ++i) to[count[((uint32_t)from[i].col >> shift) & mask]++] = from[i];
        std::swap(from, to);
    }
    if (from != E.data()) E.swap(tmp);
}

// Indices 0 .. n - 1 with size_of(i) > 0, largest first, equal sizes in index order (a counting sort: sizes are
// mostly small; the few above the table are sorted by comparison).
template <typename Size>
std::vector<int> largest_first(int n, Size size_of)
{
    constexpr long long kTable = 1 << 16;
    std::vector<int> count((size_t)kTable + 1, 0), big, order;
    for (int i = 0; i < n; ++i) {
        const long long s = size_of(i);
        if (s >= kTable) big.push_back(i);
        else if (s > 0) ++count[(size_t)s];
    }
    std::stable_sort(big.begin(), big.end(), [&](int a, int b) { return size_of(a) > size_of(b); });
    // first place of every size among the small ones, largest size first
    long long at = (long long)big.size();
    for (long long s = kTable - 1; s >= 1; --s) {
        const int c = count[(size_t)s];
        count[(size_t)s] = (int)at;
        at += c;
    }
    order.resize((size_t)at);
    std::copy(big.begin(), big.end(), order.begin());
    for (int i = 0; i < n; ++i) {
        const long long s = size_of(i);
        if (s > 0 && s < kTable) order[(size_t)count[(size_t)s]++] = i;
    }
    return order;
}

// Largest first, each to the bin with the smallest load so far; a bin takes at most `cap` of `cost`.
// load, used: per bin, what it holds before (may be null: nothing) and after.  false if some item finds no bin.
template <typename Size, typename Cost>
bool deal_largest_first(const int *order, size_t count, Size size_of, Cost cost_of, int bins, long long cap, std::vector<int> &bin_of,
                        long long *load = nullptr, long long *used_io = nullptr)
{
    typedef std::pair<long long, int> Load;  // (load, bin): the lightest bin first, the lower index among equals
    std::priority_queue<Load, std::vector<Load>, std::greater<Load>> heap;
    for (int b = 0; b < bins; ++b) heap.push(Load(load ? load[b] : 0, b));
    std::vector<long long> used((size_t)bins, 0);
    if (used_io) used.assign(used_io, used_io + bins);
    std::vector<Load> held;
    for (size_t k = 0; k < count; ++k) {
        const int i = order[k];
        held.clear();
        Load top;
        for (;;) {
            if (heap.empty()) return false;
            top = heap.top();
            heap.pop();
            if (used[(size_t)top.second] + cost_of(i) <= cap) break;
            held.push_back(top);
        }
        for (const Load &h : held) heap.push(h);
        bin_of[(size_t)i] = top.second;
        used[(size_t)top.second] += cost_of(i);
        heap.push(Load(top.first + size_of(i), top.second));
    }
    if (load)
        for (; !heap.empty(); heap.pop()) load[heap.top().second] = heap.top().first;
    if (used_io) std::copy(used.begin(), used.end(), used_io);
    return true;
}

template <typename Size, typename Cost>
bool deal_largest_first(const std::vector<int> &order, Size size_of, Cost cost_of, int bins, long long cap, std::vector<int> &bin_of)
{
    return deal_largest_first(order.data(), order.size(), size_of, cost_of, bins, cap, bin_of);
}

}  // namespace

int plan_panels(const int *rp, int n, int nnz, int K, const BuildParams &bp, Layout &out, Bulk<ListedRow> &listed_rows)
{
    if (n < 1 || nnz < 0 || K < 1 || !rp) return MPS_ERR_INVALID_ARG;
    if (bp.elem_bytes != 4 && bp.elem_bytes != 2) return MPS_ERR_INVALID_ARG;
    const long long row_bytes = (long long)K * bp.elem_bytes;
    if (row_bytes % 4 != 0) return MPS_ERR_UNSUPPORTED;  // (an odd number of halves: rows of X that start between two dwords)
    // Rows of up to 64 bytes: one tile of 4 lanes; wider ones: tiles of 8 lanes (128 bytes), the last of them as wide as
    // what is left of the row - lanes past the row's end add up bytes that nobody reads.
    const int L = row_bytes <= 64 ? 4 : 8;
    const int tiles = (int)((row_bytes + 16 * L - 1) / (16 * L));
    const int acc_row_bytes = 16 * L * (4 / bp.elem_bytes);  // fp32 sums of a tile: 16 L bytes of floats, 32 L of halves
    const int col_bits = bits_for((unsigned)(n - 1));
    if (col_bits > 32 - kMinRowBits) return MPS_ERR_UNSUPPORTED;
    const int num_cus = bp.num_cus > 0 ? bp.num_cus : 256;
    long long vcap = (kLdsBytes - 1024) / acc_row_bytes - 1;           // one row for the padding's sums
    vcap = std::min<long long>(vcap, (1ll << (32 - col_bits)) - 2);
    if (bp.acc_rows > 0) vcap = std::min<long long>(vcap, bp.acc_rows);
    vcap &= ~3ll;
    if (vcap < 4) return MPS_ERR_UNSUPPORTED;
    const int U = row_bytes <= 64 ? 2 : 1;  // rows of Y per 128-byte line

    out = Layout();
    out.n = n;
    out.nnz = nnz;
    out.K = K;
    out.elem_bytes = bp.elem_bytes;
    out.lanes = L;
    out.tiles = tiles;
    out.col_bits = col_bits;
    out.bank_rows = std::max(1, 256 / (16 * L));
    const int gpw = 64 / L;  // lane-groups of a wavefront = entries of an instruction
    // instructions whose entries are added up at the same time (see Layout::together).  Measured on MI355X, R-MAT
    // scale 20 / 22, ms per product with 1 / 2: 64-byte rows 0.1285 / 0.1278; 128-byte tiles 0.167 / 0.168 (K = 256:
    // 1.358 / 1.384); fp16 rows of 128 bytes 0.934 / 0.960 (what pairs save on LDS round trips, their 4 % more padding
    // costs again).
    const int together = bp.together > 0 ? bp.together : (L == 4 ? 2 : 1);
    if (together != 1 && together != 2) return MPS_ERR_INVALID_ARG;
    out.together = together;

    auto deg = [&](int r) { return (long long)rp[r + 1] - rp[r]; };

    // ---- panels: how many, how rows are cut, which row goes where
    Bulk<Item> items;  // (filled chunk by chunk on all threads: not zeroed first)
    std::vector<int> item_panel, order;  // order: the items that hold nonzeros, largest first
    std::vector<int> split_of((size_t)n, 0);  // sub-rows of a row (0: not split)
    int NP = 0, piece = 0;
    // rows per degree: what a number of panels needs in accumulator rows is summed over these, not over the rows
    std::vector<std::pair<long long, long long>> by_degree;  // (degree, rows), degrees in ascending order
    {
        constexpr long long kSmall = 1 << 16;
        std::vector<long long> small((size_t)kSmall, 0), large;
        for (int r = 0; r < n; ++r) {
            const long long d = deg(r);
            if (d < kSmall) ++small[(size_t)d]; else large.push_back(d);
        }
        for (long long d = 0; d < kSmall; ++d)
            if (small[(size_t)d]) by_degree.emplace_back(d, small[(size_t)d]);
        std::sort(large.begin(), large.end());
        for (size_t i = 0; i < large.size();) {
            size_t j = i;
            while (j < large.size() && large[j] == large[i]) ++j;
            by_degree.emplace_back(large[i], (long long)(j - i));
            i = j;
        }
    }
    for (int R = 1;; ++R) {
        if (R > 8192) return MPS_ERR_UNSUPPORTED;  // (a row that needs more accumulator rows than a panel holds)
        NP = num_cus * R;
        const long long share = std::max<long long>(1, (long long)nnz / NP);
        // An accumulator row takes one entry per instruction (or pair of instructions) at most, and a wavefront's
        // share is share / 16 / gpw instructions: a piece of half that many entries finds its places among them
        // (R-MAT scale 20, 16 per row: 1 % padding with one instruction at a time, 5 % with pairs; pieces of half
        // the size need half as many accumulator rows again, and a third more panels).
        piece = bp.piece > 0 ? bp.piece : (int)std::min<long long>(1 << 20, std::max<long long>(8, share / kWaves / gpw / 2));
        // a row of about a panel's share or more is cut into sub-rows of a third of a share
        const long long split_from = std::max<long long>(share - share / 10, 4ll * piece);
        const long long sub_target = std::max<long long>(share / 3, piece);
        auto pieces_of = [&](long long d) { return (int)((d + piece - 1) / piece); };
        auto sub_rows_of = [&](long long d) {
            const int S = d > split_from && NP > 1 ? (int)((d + sub_target - 1) / sub_target) : 0;
            return S == 1 ? 0 : S;
        };
        {
            long long need = 0;  // accumulator rows in all
            for (const auto &dc : by_degree) {
                const long long d = dc.first;
                const int S = sub_rows_of(d);
                long long p = 0;
                if (S > 0) {
                    for (int j = 0; j < S; ++j) p += pieces_of(d / S + (j < d % S));
                } else {
                    p = pieces_of(d);
                }
                need += p * dc.second;
            }
            if (need > (long long)NP * vcap) continue;
        }
        // the items, in row order: the rows in chunks that start at even rows (so that pairs never span two chunks),
        // every chunk on its own, then one after the other
        mps_host::parallel_for(n, 1 << 16, [&](int64_t lo, int64_t hi) {
            for (int64_t r = lo; r < hi; ++r) split_of[(size_t)r] = sub_rows_of(deg((int)r));
        });
        constexpr int kChunkRows = 1 << 16;
        const int chunks = (n + kChunkRows - 1) / kChunkRows;
        std::vector<std::vector<Item>> chunk_items((size_t)chunks);
        std::vector<std::vector<int>> chunk_split((size_t)chunks);
        mps_host::parallel_for(chunks, 1, [&](int64_t c0, int64_t c1) {
            for (int64_t c = c0; c < c1; ++c) {
                std::vector<Item> &mine = chunk_items[(size_t)c];
                const int r_end = (int)std::min<long long>(n, (c + 1) * (long long)kChunkRows);
                mine.reserve((size_t)kChunkRows / (size_t)U + 16);
                for (int r = (int)(c * kChunkRows); r < r_end;) {
                    const int S = split_of[(size_t)r];
                    if (S > 0) {
                        const long long d = deg(r);
                        for (int j = 0; j < S; ++j) {
                            const long long dj = d / S + (j < d % S);  // entries j, j + S, j + 2 S, ...
                            mine.push_back(Item{dj, pieces_of(dj), r, 1, j});
                        }
                        chunk_split[(size_t)c].push_back(r);
                        ++r;
                        continue;
                    }
                    int take = 1;
                    if (U == 2 && (r & 1) == 0 && r + 1 < n && split_of[(size_t)r + 1] == 0) take = 2;
                    long long d = 0;
                    int p = 0;
                    for (int k = 0; k < take; ++k) {
                        d += deg(r + k);
                        p += pieces_of(deg(r + k));
                    }
                    mine.push_back(Item{d, p, r, take, -1});
                    r += take;
                }
            }
        });
        items.clear();
        out.split_row.clear();
        out.split_ptr.assign(1, 0);
        long long totv = 0;
        {
            std::vector<size_t> first((size_t)chunks + 1, 0);
            for (int c = 0; c < chunks; ++c) first[(size_t)c + 1] = first[(size_t)c] + chunk_items[(size_t)c].size();
            items.resize(first[(size_t)chunks]);
            mps_host::parallel_for(chunks, 1, [&](int64_t c0, int64_t c1) {
                for (int64_t c = c0; c < c1; ++c)
                    std::copy(chunk_items[(size_t)c].begin(), chunk_items[(size_t)c].end(), items.begin() + (long)first[(size_t)c]);
            });
            for (int c = 0; c < chunks; ++c)
                for (int r : chunk_split[(size_t)c]) {
                    out.split_row.push_back(r);
                    out.split_ptr.push_back(out.split_ptr.back() + split_of[(size_t)r]);
                }
            std::atomic<long long> pieces{0};
            mps_host::parallel_for(chunks, 1, [&](int64_t c0, int64_t c1) {
                long long mine = 0;
                for (int64_t c = c0; c < c1; ++c)
                    for (const Item &it : chunk_items[(size_t)c]) mine += it.pieces;
                pieces.fetch_add(mine, std::memory_order_relaxed);
            });
            totv = pieces.load();
        }
        if (totv > (long long)NP * vcap) continue;
        order = largest_first((int)items.size(), [&](int i) { return items[(size_t)i].nnz; });
        item_panel.assign(items.size(), 0);
        auto nnz_of = [&](int i) { return items[(size_t)i].nnz; };
        auto pieces_needed = [&](int i) { return (long long)items[(size_t)i].pieces; };
        // Many items and many panels: the first 32 items per panel (the long rows) from one deal; then the panels in up
        // to 16 sets of at least 16, the other items (largest first) dealt to the sets in turn, and every set dealt on
        // a thread of its own from where the first deal left its panels.  The sets get the same mix of sizes, so the
        // panels end up as even as from one deal.
        const int sets = items.size() >= (size_t)100000 ? std::min(16, NP / 16) : 1;
        const size_t head = sets > 1 ? std::min(order.size(), (size_t)32 * (size_t)NP) : order.size();
        std::vector<long long> load((size_t)NP, 0), used((size_t)NP, 0);
        if (!deal_largest_first(order.data(), head, nnz_of, pieces_needed, NP, vcap, item_panel, load.data(), used.data())) continue;
        if (head < order.size()) {
            std::vector<std::vector<int>> set_order((size_t)sets);
            for (auto &o : set_order) o.reserve((order.size() - head) / (size_t)sets + 1);
            for (size_t k = head; k < order.size(); ++k) set_order[k % (size_t)sets].push_back(order[k]);
            std::atomic<bool> dealt{true};
            mps_host::parallel_for(sets, 1, [&](int64_t lo, int64_t hi) {
                for (int64_t q = lo; q < hi; ++q) {
                    const int first = (int)(q * NP / sets), bins = (int)((q + 1) * NP / sets) - first;
                    const std::vector<int> &mine = set_order[(size_t)q];
                    if (!deal_largest_first(mine.data(), mine.size(), nnz_of, pieces_needed, bins, vcap, item_panel,
                                            load.data() + first, used.data() + first))
                        dealt.store(false, std::memory_order_relaxed);
                    for (int i : mine) item_panel[(size_t)i] += first;
                }
            });
            if (!dealt.load()) continue;
        }
        // rows without nonzeros: zeros to write, dealt evenly
        int turn = 0;
        for (int i = 0; i < (int)items.size(); ++i)
            if (items[(size_t)i].nnz == 0) item_panel[(size_t)i] = turn++ % NP;
        break;
    }
    out.num_panels = NP;
    out.piece = piece;

    // a panel's items: those with nonzeros largest first, then the empty ones
    std::vector<int> panel_count((size_t)NP + 1, 0);
    for (size_t i = 0; i < items.size(); ++i) panel_count[(size_t)item_panel[i] + 1] += 1;
    for (int p = 0; p < NP; ++p) panel_count[(size_t)p + 1] += panel_count[(size_t)p];
    std::vector<int> panel_items(items.size());
    {
        std::vector<int> fill(panel_count.begin(), panel_count.end() - 1);
        for (int i : order) panel_items[(size_t)fill[(size_t)item_panel[(size_t)i]]++] = i;
        for (int i = 0; i < (int)items.size(); ++i)
            if (items[(size_t)i].nnz == 0) panel_items[(size_t)fill[(size_t)item_panel[(size_t)i]]++] = i;
    }
    // partial row of sub-row j of split row r
    std::vector<int> split_index((size_t)n, -1);
    for (size_t i = 0; i < out.split_row.size(); ++i) split_index[(size_t)out.split_row[i]] = (int)i;

    // listed rows and accumulator rows per panel
    out.panel_ptr.assign((size_t)NP + 1, 0);
    std::vector<int> panel_pieces((size_t)NP, 0);
    mps_host::parallel_for(NP, 16, [&](int64_t lo, int64_t hi) {
        for (int64_t p = lo; p < hi; ++p) {
            int rows = 0, v = 0;
            for (int k = panel_count[(size_t)p]; k < panel_count[(size_t)p + 1]; ++k) {
                rows += items[(size_t)panel_items[(size_t)k]].nrows;
                v += items[(size_t)panel_items[(size_t)k]].pieces;
            }
            out.panel_ptr[(size_t)p + 1] = rows;
            panel_pieces[(size_t)p] = v;
        }
    });
    for (int p = 0; p < NP; ++p) out.panel_ptr[(size_t)p + 1] += out.panel_ptr[(size_t)p];
    const int listed = out.panel_ptr[(size_t)NP];
    int acc_rows = 4;
    for (int p = 0; p < NP; ++p) acc_rows = std::max(acc_rows, (panel_pieces[(size_t)p] + 3) & ~3);
    out.acc_rows = acc_rows;
    out.rows.assign((size_t)listed, 0);
    out.piece_ptr.assign((size_t)listed + NP, 0);
    out.wave_meta.assign((size_t)NP * kWaves * 2, 0);
    out.panel_rounds.assign((size_t)NP, 0);

    // the listed rows of every panel: which entries of the matrix they hold and where their accumulator rows start
    listed_rows.resize((size_t)listed);
    mps_host::parallel_for(NP, 64, [&](int64_t lo, int64_t hi) {
        for (int p = (int)lo; p < (int)hi; ++p) {
            int lr = out.panel_ptr[(size_t)p];
            int *pp = out.piece_ptr.data() + lr + p;
            int v = 0;
            long long before = 0;
            for (int k = panel_count[(size_t)p]; k < panel_count[(size_t)p + 1]; ++k) {
                const Item &it = items[(size_t)panel_items[(size_t)k]];
                for (int q = 0; q < it.nrows; ++q) {
                    const int r = it.row + q;
                    const long long d = it.sub >= 0 ? it.nnz : deg(r);
                    const int P = (int)((d + piece - 1) / piece);
                    out.rows[(size_t)lr] = it.sub >= 0 ? n + out.split_ptr[(size_t)split_index[(size_t)r]] + it.sub : r;
                    ListedRow &L = listed_rows[(size_t)lr];
                    L.row = r;
                    L.first = it.sub >= 0 ? it.sub : 0;
                    L.stride = it.sub >= 0 ? split_of[(size_t)r] : 1;
                    L.entries = (int)d;
                    L.pieces = P;
                    L.first_piece = v;
                    L.entries_before = before;
                    *pp++ = v;
                    ++lr;
                    v += P;
                    before += d;
                }
            }
            *pp = v;
        }
    });
    return MPS_OK;
}

int build_streams(const int *rp, const int *ci, const float *val, const BuildParams &bp, Layout &out,
                  const Bulk<ListedRow> &listed_rows)
{
    if (out.nnz > 0 && (!ci || !val)) return MPS_ERR_INVALID_ARG;
    const int NP = out.num_panels, L = out.lanes, G = out.bank_rows, gpw = 64 / L, together = out.together, piece = out.piece;
    const int group_slots = gpw * together, col_bits = out.col_bits;
    const uint32_t pad_word = (uint32_t)out.acc_rows << col_bits;  // padding: column 0, value 0, the spare accumulator row
    (void)piece;
        // ---- every panel on its own: accumulator rows, wavefronts, streams
    struct PanelOut {
        Bulk<uint32_t> stream;
        std::vector<int> src;
        int wave_rounds[kWaves];
        int vrows;
    };
    std::vector<PanelOut> built((size_t)NP);
    const int words_per_round = gpw * kWin * 4;  // uint32: lane-groups x 4 lanes x {word A, value A, word B, value B}
    mps_host::parallel_for(NP, 1, [&](int64_t lo, int64_t hi) {
        std::vector<int> vsize, vwave, vorder, last;
        std::vector<Entry> entries[kWaves], sort_tmp;
        std::vector<int> sort_count;
        std::vector<uint8_t> fill;
        std::vector<long long> slot;
        for (int p = (int)lo; p < (int)hi; ++p) {
            PanelOut &po = built[(size_t)p];
            // the sizes of the accumulator rows
            const int l0 = out.panel_ptr[(size_t)p], l1 = out.panel_ptr[(size_t)p + 1];
            int v = 0;
            vsize.clear();
            for (int l = l0; l < l1; ++l) {
                const ListedRow &R = listed_rows[(size_t)l];
                for (int j = 0; j < R.pieces; ++j) vsize.push_back(R.entries / R.pieces + (j < R.entries % R.pieces));
                v += R.pieces;
            }
            po.vrows = v;
            // accumulator rows to wavefronts
            vorder = largest_first(v, [&](int i) { return (long long)vsize[(size_t)i]; });
            vwave.assign((size_t)v, 0);
            deal_largest_first(
                vorder, [&](int i) { return (long long)vsize[(size_t)i]; }, [](int) { return 0ll; }, kWaves, 1, vwave);
            // entries per wavefront
            for (auto &e : entries) e.clear();
            for (int l = l0; l < l1; ++l) {
                const ListedRow &R = listed_rows[(size_t)l];
                const long long base = rp[R.row];
                for (long long e = 0; e < R.entries; ++e) {
                    const long long at = base + R.first + e * R.stride;
                    const int vl = R.first_piece + (int)(e % R.pieces);
                    entries[vwave[(size_t)vl]].push_back(Entry{ci[at], vl, val[at], (int)at});
                }
            }
            // streams: a wavefront's entries by column; one entry per lane-group and instruction, never two of one
            // accumulator row in an instruction (the second waits for the next instruction that has room)
            for (int w = 0; w < kWaves; ++w) {
                std::vector<Entry> &E = entries[w];
                sort_by_column(E, sort_tmp, sort_count, col_bits);
                const long long ne = (long long)E.size();
                slot.resize((size_t)ne);
                fill.assign((size_t)(ne / group_slots + 2), 0);
                last.assign((size_t)po.vrows + 1, -1);
                long long frontier = 0, top = 0;
                for (long long e = 0; e < ne; ++e) {
                    const int vl = E[(size_t)e].vloc;
                    long long t = std::max<long long>(frontier, (long long)last[(size_t)vl] + 1);
                    for (;;) {
                        if (t >= (long long)fill.size()) fill.resize((size_t)t + ne / group_slots + 2, 0);
                        if (fill[(size_t)t] < group_slots) break;
                        ++t;
                    }
                    slot[(size_t)e] = t * group_slots + fill[(size_t)t];
                    ++fill[(size_t)t];
                    last[(size_t)vl] = (int)t;
                    top = std::max(top, t + 1);
                    while (frontier < (long long)fill.size() && fill[(size_t)frontier] == group_slots) ++frontier;
                }
                const int groups_per_round = kRoundInstr / together;
                const int rounds = (int)((top + groups_per_round - 1) / groups_per_round);
                po.wave_rounds[w] = rounds;
                const size_t at0 = po.stream.size();
                po.stream.resize(at0 + (size_t)rounds * words_per_round);
                if (bp.keep_src) po.src.resize((at0 + (size_t)rounds * words_per_round) / 2, -1);
                uint32_t *s = po.stream.data() + at0;
                for (size_t i = 0; i < (size_t)rounds * words_per_round; i += 2) {
                    s[i] = pad_word;
                    s[i + 1] = 0u;
                }
                for (long long e = 0; e < ne; ++e) {
                    // group t, place i in it -> round, window (A / B), lane of the quad, lane-group: a group is one
                    // instruction, or entry q of both windows
                    const long long t = slot[(size_t)e] / group_slots, i = slot[(size_t)e] % group_slots;
                    const long long round = t / groups_per_round, g = i % gpw;
                    const long long w2 = together == 2 ? i / gpw : (t % kRoundInstr) / kWin, q = t % kWin;
                    const size_t at = (size_t)((round * gpw * kWin + g * kWin + q) * 4 + w2 * 2);
                    uint32_t bits;
                    std::memcpy(&bits, &E[(size_t)e].val, 4);
                    s[at] = (uint32_t)E[(size_t)e].col | ((uint32_t)swizzle(E[(size_t)e].vloc, G) << col_bits);
                    s[at + 1] = bits;
                    if (bp.keep_src) po.src[(at0 + at) / 2] = E[(size_t)e].src;
                }
            }
        }
    });

    // ---- put the panels' streams one after the other
    std::vector<long long> panel_first((size_t)NP + 1, 0);
    for (int p = 0; p < NP; ++p) {
        long long rounds = 0;
        int most = 0;
        for (int w = 0; w < kWaves; ++w) {
            out.wave_meta[((size_t)p * kWaves + w) * 2] = (int)(panel_first[(size_t)p] + rounds);
            out.wave_meta[((size_t)p * kWaves + w) * 2 + 1] = built[(size_t)p].wave_rounds[w];
            rounds += built[(size_t)p].wave_rounds[w];
            most = std::max(most, built[(size_t)p].wave_rounds[w]);
        }
        out.panel_rounds[(size_t)p] = most;
        panel_first[(size_t)p + 1] = panel_first[(size_t)p] + rounds;
    }
    out.rounds = panel_first[(size_t)NP];
    if (out.rounds * (long long)words_per_round / 4 > 0x7fffffffll) return MPS_ERR_UNSUPPORTED;  // 16-byte units index the stream
    out.stream.resize((size_t)out.rounds * words_per_round);
    if (bp.keep_src) out.src.resize(out.stream.size() / 2);
    mps_host::parallel_for(NP, 1, [&](int64_t lo, int64_t hi) {
        for (int p = (int)lo; p < (int)hi; ++p) {
            PanelOut &po = built[(size_t)p];
            if (!po.stream.empty())
                std::memcpy(out.stream.data() + (size_t)panel_first[(size_t)p] * words_per_round, po.stream.data(),
                            po.stream.size() * sizeof(uint32_t));
            if (bp.keep_src && !po.src.empty())
                std::memcpy(out.src.data() + (size_t)panel_first[(size_t)p] * words_per_round / 2, po.src.data(),
                            po.src.size() * sizeof(int));
            Bulk<uint32_t>().swap(po.stream);
            std::vector<int>().swap(po.src);
        }
    });
    return MPS_OK;
}

int build_layout(const int *rp, const int *ci, const float *val, int n, int nnz, int K, const BuildParams &bp, Layout &out)
{
    if (nnz > 0 && (!ci || !val)) return MPS_ERR_INVALID_ARG;
    Bulk<ListedRow> listed_rows;
    const int rc = plan_panels(rp, n, nnz, K, bp, out, listed_rows);
    return rc != MPS_OK ? rc : build_streams(rp, ci, val, bp, out, listed_rows);
}

}  // namespace mps_sw

struct mps_sweep_layout {
    mps_sw::Layout L;
};

extern "C" {

int mps_sweep_layout_build(const int *row_ptr, const int *col_idx, const float *val, int n_rows, int nnz, int K,
                           int elem_bytes, const mps_plan_options *options, mps_sweep_layout **layout_out)
{
    if (!layout_out) return MPS_ERR_INVALID_ARG;
    *layout_out = nullptr;
    mps_sw::BuildParams bp;
    bp.elem_bytes = elem_bytes;
    if (options) {
        bp.piece = options->sweep_piece;
        bp.acc_rows = options->sweep_acc_rows;
        bp.num_cus = options->sweep_panels_per_round;
        bp.together = options->sweep_together;
        bp.keep_src = !(options->flags & MPS_PLAN_NO_SOURCES);
    }
    if (bp.num_cus <= 0) bp.num_cus = 256;
    mps_sweep_layout *h = new (std::nothrow) mps_sweep_layout;
    if (!h) return MPS_ERR_UNSUPPORTED;
    int rc;
    try {
        rc = mps_sw::build_layout(row_ptr, col_idx, val, n_rows, nnz, K, bp, h->L);
    } catch (const std::bad_alloc &) {
        rc = MPS_ERR_UNSUPPORTED;
    }
    if (rc != MPS_OK) {
        delete h;
        return rc;
    }
    *layout_out = h;
    return MPS_OK;
}

}  // extern "C"

namespace mps_sw {
void fill_info(const Layout &L, mps_plan_info *info)
{
    info->sweep_panels = L.num_panels;
    info->sweep_acc_rows = L.acc_rows;
    info->sweep_lanes = L.lanes;
    info->sweep_tiles = L.tiles;
    info->sweep_col_bits = L.col_bits;
    info->sweep_piece = L.piece;
    info->sweep_together = L.together;
    info->sweep_split_rows = (int)L.split_row.size();
    info->sweep_partial_rows = L.split_ptr.empty() ? 0 : L.split_ptr.back();
    info->sweep_listed_rows = (int)L.rows.size();
    info->sweep_rounds = L.rounds;
    info->sweep_slots = L.rounds * (long long)(64 / L.lanes) * kRoundInstr;
}
}  // namespace mps_sw

extern "C" {

int mps_sweep_layout_info(const mps_sweep_layout *layout, mps_plan_info *info)
{
    if (!layout || !info) return MPS_ERR_INVALID_ARG;
    const mps_sw::Layout &L = layout->L;
    std::memset(info, 0, sizeof(*info));
    info->n_rows = L.n;
    info->nnz = L.nnz;
    info->K = L.K;
    info->elem_bytes = L.elem_bytes;
    info->num_slabs = 1;
    info->slab_cols = L.n;
    mps_sw::fill_info(L, info);
    return MPS_OK;
}

int mps_sweep_layout_array(const mps_sweep_layout *layout, int which, const void **data_out, size_t *bytes_out)
{
    if (!layout || !data_out || !bytes_out) return MPS_ERR_INVALID_ARG;
    const mps_sw::Layout &L = layout->L;
    auto give = [&](const auto &v) {
        *data_out = v.data();
        *bytes_out = v.size() * sizeof(v[0]);
        return (int)MPS_OK;
    };
    switch (which) {
    case MPS_PLAN_ARRAY_SW_PANEL_PTR: return give(L.panel_ptr);
    case MPS_PLAN_ARRAY_SW_ROWS: return give(L.rows);
    case MPS_PLAN_ARRAY_SW_PIECE_PTR: return give(L.piece_ptr);
    case MPS_PLAN_ARRAY_SW_WAVE_META: return give(L.wave_meta);
    case MPS_PLAN_ARRAY_SW_PANEL_ROUNDS: return give(L.panel_rounds);
    case MPS_PLAN_ARRAY_SW_STREAM: return give(L.stream);
    case MPS_PLAN_ARRAY_SW_SRC: return give(L.src);
    case MPS_PLAN_ARRAY_SW_SPLIT_ROW: return give(L.split_row);
    case MPS_PLAN_ARRAY_SW_SPLIT_PTR: return give(L.split_ptr);
    default: return MPS_ERR_INVALID_ARG;
    }
}

void mps_sweep_layout_free(mps_sweep_layout *layout) { delete layout; }

}  // extern "C"
