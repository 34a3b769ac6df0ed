// Host-side builder of row-block plans (layout described in
// mpspmm_rowblock.hpp).  Pure host code: no GPU is touched here.
#include "mpspmm_rowblock.hpp"

#include <algorithm>
#include <atomic>
#include <cstring>
#include <new>

#include "mpspmm.h"
#include "mpspmm_hostpar.hpp"

namespace mps_rb {

namespace {

using mps_host::parallel_for;

// Contiguous row blocks of at most `cap` rows and (except for a single row
// that is longer) at most `target` nonzeros each, taken greedily.
int greedy_blocks(const int *rp, int n, int cap, long long target, std::vector<int> *out)
{
    int count = 0, r = 0;
    if (out) out->assign(1, 0);
    while (r < n) {
        const int hi = (int)std::min<long long>(n, (long long)r + cap);
        // furthest e in (r, hi] with rp[e] - rp[r] <= target
        const long long limit = (long long)rp[r] + target;
        int e = (int)(std::upper_bound(rp + r + 1, rp + hi + 1, limit,
                                       [](long long lim, int v) { return lim < (long long)v; }) -
                      rp) - 1;
        if (e <= r) e = r + 1;
        r = e;
        ++count;
        if (out) out->push_back(r);
    }
    return count;
}

inline int windows_of(int entries) { return (entries + kWin - 1) / kWin; }

// Everything about one (block, step): where each wavefront's run starts.
struct StepSplit {
    int first_row[kWaves];
    int hstart[kWaves + 1], cstart[kWaves + 1];
    int cut[kWaves + 1];  // windows of the step (hot and cold, row order) before the run
};

// cnt_t: [lr * 2 + kind] nonzeros of local row lr in this step (kind 0 hot, 1 cold).  The step's
// windows in row order (a row's hot windows, then its cold ones) are cut into 16 runs (see kCutSlack).
void split_step(const int *cnt_t, int nr, StepSplit &sp, std::vector<int> &before)
{
    // before[lr * 2 + kind]: windows of the kind in the rows before lr
    before.resize((size_t)2 * nr + 2);
    int hot_total = 0, cold_total = 0;
    for (int lr = 0; lr < nr; ++lr) {
        before[(size_t)2 * lr] = hot_total;
        before[(size_t)2 * lr + 1] = cold_total;
        hot_total += windows_of(cnt_t[2 * lr]);
        cold_total += windows_of(cnt_t[2 * lr + 1]);
    }
    before[(size_t)2 * nr] = hot_total;
    before[(size_t)2 * nr + 1] = cold_total;
    const long long E = (long long)hot_total + cold_total;
    // the row that holds window q of the step (q < E), and the hot and cold windows in front of q
    int at = 0;  // (the cuts never go back: the search starts where the last one ended)
    auto locate = [&](long long q, int *hot, int *cold) {
        while ((long long)before[(size_t)2 * (at + 1)] + before[(size_t)2 * (at + 1) + 1] <= q) ++at;
        const int hq = before[(size_t)2 * at], cq = before[(size_t)2 * at + 1], h = before[(size_t)2 * (at + 1)] - hq;
        const long long d = q - hq - cq;
        *hot = d < h ? hq + (int)d : hq + h;
        *cold = d < h ? cq : cq + (int)(d - h);
        return at;
    };
    const long long slack = E / kWaves / kCutSlack;
    sp.cut[0] = 0;
    sp.hstart[0] = sp.cstart[0] = 0;
    sp.first_row[0] = 0;
    if (E > 0) {
        int h0, c0;
        sp.first_row[0] = locate(0, &h0, &c0);
    }
    for (int w = 1; w < kWaves; ++w) {
        if (E == 0) {  // nothing to cut
            sp.cut[w] = sp.hstart[w] = sp.cstart[w] = 0;
            sp.first_row[w] = 0;
            continue;
        }
        const long long equal_cut = (long long)w * E / kWaves;
        const long long lo = std::max<long long>(sp.cut[w - 1], equal_cut - slack), hi = std::min(equal_cut + slack, E - 1);
        unsigned long long best = ~0ull;
        const int at0 = at;
        for (long long q = lo; q <= hi; ++q) {
            int hot, cold;
            locate(q, &hot, &cold);
            best = std::min(best, cut_key(hot - sp.hstart[w - 1], cold - sp.cstart[w - 1], q, equal_cut));
        }
        at = at0;
        const long long q = (long long)(best & 0xffffffffull);
        sp.cut[w] = (int)q;
        sp.first_row[w] = locate(q, &sp.hstart[w], &sp.cstart[w]);
    }
    sp.cut[kWaves] = (int)E;
    sp.hstart[kWaves] = hot_total;
    sp.cstart[kWaves] = cold_total;
}

void count_block(const int *rp, const int *ci, const ColumnMap &cm, int b, int r0, int nr, int T, std::vector<int> &cnt)
{
    cnt.assign((size_t)T * nr * 2, 0);
    for (int lr = 0; lr < nr; ++lr)
        for (int e = rp[r0 + lr]; e < rp[r0 + lr + 1]; ++e) {
            const int c = ci[e];
            ++cnt[((size_t)cm.step_of(b, c) * nr + lr) * 2 + (cm.slot_of(b, c) < 0)];
        }
}

}  // namespace

int default_steps(int n, long long nnz, int table_rows, int num_blocks, const long long *table_nnz, int tables)
{
    // table_nnz[k]: nonzeros in the columns that a (k + 1)-th table would serve (ranks k H .. (k + 1) H - 1 by
    // nonzero count), for k < tables.  Every step costs a block two barriers, a table load and some padded windows
    // (about 3 us on MI355X, the time of 3,000 nonzeros).  Two things ask for steps, and the larger one decides.
    // (1) The range of X that a step gathers through L2 should stay in the 4 MiB L2 of an XCD: 5 MiB of X per step
    //     where the columns are skewed (the busy part of a range stays), 3 MiB where they are not - but no more
    //     steps than leave a block 7,000 (skewed) or 5,000 nonzeros each: below that the steps cost more than the
    //     L2 misses they save.
    // (2) Tables: every step puts another H columns into LDS.  A block wants about 28,000 nonzeros per step, and a
    //     table is worth its step while it serves 1 % of the nonzeros.
    // Measured on MI355X (ms per product at 2 / 3 / 4 / 6 / 8 / 12 / 16 steps; in brackets what this rule picks):
    //   power law,   232,965 rows x  32 per row: .057 .055 .057 .066 .077 .090  -       (3)
    //   power law,   232,965 rows x  64:         .095 .083 .081 .086 .098 .117 .142     (3)
    //   power law,   232,965 rows x 128:         .175 .151 .148 .145 .149 .163 .188     (4)
    //   power law,   232,965 rows x 200:         .271 .235 .224 .212 .210 .220 .235     (7)
    //   power law,   232,965 rows x 492:         13 to 18 steps within 1.5 % of each other (16)
    //   power law,   500,000 rows x  64:         .280 .245 .231 .226 .232 .257 .301     (7)
    //   power law,   500,000 rows x 200:         .864 .712 .629 .560 .546 .546 .547     (7)
    //   power law, 1,000,000 rows x  64:         .721 .662 .635 .604 .577 .573 .636     (8)
    //   power law, 1,000,000 rows x 128:         1.45 1.31 1.21 1.12 1.06 1.04 1.01     (13)
    //   power law, 1,000,000 rows x  32 (2, 4, 6, 8, 13 steps): .361 .336 .330 .351 .457                    (4)
    //   power law, 1,000,000 rows x  16 (1, 2, 3, 4, 13 steps): .216 .202 .199 .203 .331                    (2)
    //   power law,   500,000 rows x  16 (2, 4 steps):           .089 .096                                   (2)
    //   R-MAT scale 20, 16 per row (1, 2, 3, 4, 6, 8, 13):      .184 .190 .190 .207 .247 .290 .378          (1)
    //   R-MAT scale 18, 16 per row (1, 2, 4):                   .046 .053 .067                              (1)
    //   uniform,     232,965 rows x 100 (2, 3, 4, 6, 10, 13 steps): .220 .164 .151 .148 .159 .167   (5)
    //   uniform,     232,965 rows x 300:                            .610 .480 .418 .414 .415 .419   (5)
    //   uniform,     500,000 rows x  64:                            .448 .389 .339 .283 .280 .296   (11)
    //   uniform,   1,000,000 rows x 100:                            1.64 1.49 1.37 1.19 .946 .921   (19)
    //   uniform,   1,000,000 rows x  60 (6, 10, 14, 21 steps):      .762 .648 .658 .795             (11)
    // Never more table slots than columns.
    if (table_rows < 1) table_rows = 1;
    if (num_blocks < 1) num_blocks = 1;
    const bool skewed = tables > 0 && nnz > 0 && (double)table_nnz[0] >= 0.05 * (double)nnz;
    const long long per_step = skewed ? (5ll << 20) : (3ll << 20);
    long long for_l2 = ((long long)n * 64 + per_step - 1) / per_step;
    for_l2 = std::min(for_l2, nnz / num_blocks / (skewed ? 7000 : 5000));
    long long for_tables = (nnz / num_blocks + 14000) / 28000;
    if (for_tables > tables) for_tables = tables;
    while (for_tables > 0 && (double)table_nnz[for_tables - 1] < 0.01 * (double)nnz) --for_tables;
    long long t = std::min<long long>(std::max(for_tables, for_l2), 32);
    const long long most = ((long long)n + table_rows - 1) / table_rows;
    if (t > most) t = most;
    return (int)std::max<long long>(t, 1);
}

int plan_blocks(const int *rp, int n, int nnz, const BuildParams &bp, Layout &L, int *table_rows)
{
    if (!rp || n < 1 || nnz < 0) return MPS_ERR_INVALID_ARG;
    const int cold_bits = bits_for(n > 1 ? n - 1 : 1);
    if (cold_bits > 22) return MPS_ERR_UNSUPPORTED;
    const int num_cus = bp.num_cus > 0 ? bp.num_cus : 256;
    L = Layout();
    L.n = n;
    L.nnz = nnz;
    L.K = 16;
    L.cold_bits = cold_bits;

    // ---- 1. row blocks: about equal nonzero counts, as few rounds of workgroups as the LDS allows
    const int budget_rows = (kLdsBytes - kSlotBytes - 256) / 64;  // table rows + accumulator rows
    int cap_limit = std::min(1024, 1 << (32 - cold_bits));                      // rows_advanced must fit above the index
    if (bp.table_rows > 0) cap_limit = std::min(cap_limit, budget_rows - bp.table_rows);
    if (cap_limit < 4) return MPS_ERR_INVALID_ARG;
    int cap = bp.block_rows > 0 ? std::min(bp.block_rows, cap_limit) : cap_limit;
    if (cap < 1) cap = 1;
    // Workgroups run one to a CU and start in order of their index as CUs come free.  As few rounds of num_cus
    // blocks as the row limit allows are best (every further round costs about 5 us and 3 us per step: power law,
    // 500,000 rows x 16, 2 steps: .089 / .103 / .111 ms with 512 / 768 / 1,024 blocks), unless the row limit leaves
    // the blocks of that round far from equal: R-MAT of 2^18 rows in 256 blocks of exactly 1,024 has 11 % of the
    // nonzeros in the first (0.85 ms a product, 0.105 with 512 blocks; 768: 0.136).  Then rounds are added until no
    // block is more than half above its share, or the largest block is a single row.
    long long longest_row = 0;
    for (int r = 0; r < n; ++r) longest_row = std::max<long long>(longest_row, (long long)rp[r + 1] - rp[r]);
    // A row is never cut across blocks: a matrix whose longest row outweighs the share of a CU several times is for
    // the merge-path split of the slab plans (power law, 262,144 rows x 4 with a row of 50,000: .053 against .034 ms).
    if (bp.max_longest_row > 0.0 && (double)longest_row > bp.max_longest_row * (double)nnz / num_cus) return kNotWorthwhile;
    long long best_target = 0;
    for (int m = 1, tried = 0; tried < 8; ++m) {
        const long long most = (long long)num_cus * m;
        if (((long long)n + cap - 1) / cap > most) continue;
        long long lo = std::max<long long>(1, ((long long)nnz + most - 1) / most), hi = std::max<long long>(nnz, 1);
        const long long even = lo;
        if (greedy_blocks(rp, n, cap, hi, nullptr) > most) continue;  // cannot happen: rows alone fit
        while (lo < hi) {
            const long long mid = lo + (hi - lo) / 2;
            if (greedy_blocks(rp, n, cap, mid, nullptr) <= most) hi = mid; else lo = mid + 1;
        }
        best_target = lo;
        if (lo <= even + even / 2 || lo <= longest_row) break;
        ++tried;
    }
    greedy_blocks(rp, n, cap, best_target, &L.block_row);
    L.num_blocks = (int)L.block_row.size() - 1;
    int most_rows = 1;
    for (int b = 0; b < L.num_blocks; ++b) most_rows = std::max(most_rows, L.block_row[b + 1] - L.block_row[b]);
    L.acc_rows = (most_rows + 3) / 4 * 4;

    // ---- 2. table size, steps
    int H = bp.table_rows > 0 ? bp.table_rows : std::min(kMaxTableRows, budget_rows - L.acc_rows);
    if (H > kMaxTableRows) H = kMaxTableRows;
    *table_rows = H;
    return MPS_OK;
}

int plan_columns(const int *rp, const int *ci, int n, int nnz, const BuildParams &bp, Layout &L, int H, const int *deg,
                 const std::function<void(int, long long *, long long *)> &block_ranges, ColumnMap &cm)
{
    // ---- 3. nonzeros per column; the steps; hot columns by rank, cold columns by id range
    auto d_of = [&](int c) { return deg[(size_t)c]; };
    // the columns that hold nonzeros, busiest first, equally busy ones by id
    std::vector<int> cand;
    auto hotter = [&](int a, int b) {
        const int da = d_of(a), db = d_of(b);
        return da != db ? da > db : a < b;
    };
    int most = 0;
    for (int c = 0; c < n; ++c) most = std::max(most, d_of(c));
    const bool counted = (long long)most <= 4ll * n + 1024;  // one bucket per count: all of them in order, in two passes
    if (counted) {
        std::vector<int> first((size_t)most + 2, 0);  // first[d]: where the columns with d nonzeros start
        for (int c = 0; c < n; ++c)
            if (d_of(c) > 0) ++first[(size_t)d_of(c)];
        int at = 0;
        for (int d = most; d >= 1; --d) {
            const int here = first[(size_t)d];
            first[(size_t)d] = at;
            at += here;
        }
        cand.resize((size_t)at);
        for (int c = 0; c < n; ++c)
            if (d_of(c) > 0) cand[(size_t)first[(size_t)d_of(c)]++] = c;
    } else {
        cand.reserve((size_t)n);
        for (int c = 0; c < n; ++c)
            if (d_of(c) > 0) cand.push_back(c);
    }
    // what every further table would serve, for as many tables as a plan may get
    constexpr int kMostTables = 32;
    long long table_nnz[kMostTables] = {0};
    const size_t top = std::min<size_t>((size_t)kMostTables * H, cand.size());
    if (!counted) {
        if (top < cand.size()) std::nth_element(cand.begin(), cand.begin() + (long)top, cand.end(), hotter);
        std::sort(cand.begin(), cand.begin() + (long)top, hotter);
    }
    for (size_t k = 0; k < top; ++k) table_nnz[k / (size_t)H] += d_of(cand[k]);
    int T = bp.steps;
    if (T <= 0) T = default_steps(n, nnz, H, L.num_blocks, table_nnz, (int)((top + (size_t)H - 1) / (size_t)H));
    if (T > 4096) T = 4096;
    bool local = false;
    if (bp.max_local_share < 1.0 && nnz > 0 && !bp.local_tables) {
        // Columns near the diagonal (banded, block-diagonal): a block finds its nonzeros in one or two column
        // ranges of its own and idles through the other steps, while a plan without steps finds such an X in L2
        // anyway.  Share of the nonzeros in each block's busiest of R equal column ranges, beyond what the busiest
        // range has of the whole matrix (which is skew, not locality).
        long long own = 0, busiest = 0;
        block_ranges(std::max(T, 4), &own, &busiest);
        if ((double)(own - busiest) > bp.max_local_share * (double)nnz) local = true;
    }
    if (bp.local_tables) local = true;
    if (local && !ci) return kNeedHost;  // local tables are laid out from the column indices themselves
    if (local) {
        // Local tables: block b's table of step t holds the H consecutive columns from base[b] + t H - for a
        // block-diagonal or banded matrix nearly all of the block's nonzeros, gathered from LDS, and a table is one
        // contiguous read of X.  As many steps as the blocks' column spans need tables (the span that holds all but
        // the outer 5 % of a block's nonzeros; nine blocks in ten must fit), 8 at most; base[b] is where a window of
        // T H columns holds the most of the block's nonzeros.  Worth it where the tables serve most of the
        // nonzeros; a wider band stays with the slab plans.
        if (bp.table_rows <= 0) H = std::min(H, (n + 3) / 4 * 4);
        // a block's column indices in ascending order: counted where they span few columns (what local tables are
        // for), sorted otherwise
        auto columns_in_order = [&](int e0, int e1, std::vector<int> &cols, std::vector<int> &count) {
            cols.clear();
            if (e1 == e0) return;
            const auto ends = std::minmax_element(ci + e0, ci + e1);
            const int c_min = *ends.first;
            const long long range = (long long)*ends.second - c_min + 1;
            if (range <= 4ll * (e1 - e0) + 1024) {
                count.assign((size_t)range, 0);
                for (int e = e0; e < e1; ++e) ++count[(size_t)(ci[e] - c_min)];
                cols.reserve((size_t)(e1 - e0));
                for (long long c = 0; c < range; ++c) cols.insert(cols.end(), (size_t)count[(size_t)c], c_min + (int)c);
            } else {
                cols.assign(ci + e0, ci + e1);
                std::sort(cols.begin(), cols.end());
            }
        };
        std::vector<int> span((size_t)L.num_blocks, 1);
        parallel_for(L.num_blocks, 8, [&](int64_t b0, int64_t b1) {
            std::vector<int> cols, count;
            for (int64_t b = b0; b < b1; ++b) {
                const int e0 = rp[L.block_row[(size_t)b]], e1 = rp[L.block_row[(size_t)b + 1]];
                if (e1 == e0) continue;
                columns_in_order(e0, e1, cols, count);
                const size_t lo = cols.size() / 40, hi = cols.size() - 1 - cols.size() / 40;
                span[(size_t)b] = cols[hi] - cols[lo] + 1;
            }
        });
        T = bp.steps;
        if (T <= 0) {
            std::vector<int> sorted(span);
            const size_t at = sorted.size() - 1 - sorted.size() / 10;
            std::nth_element(sorted.begin(), sorted.begin() + (long)at, sorted.end());
            T = std::max(1, std::min(8, (sorted[at] + H - 1) / H));
        }
        T = std::max(1, std::min(T, (n + H - 1) / H));
        const long long W = (long long)T * H;
        L.table_base.assign((size_t)L.num_blocks, 0);
        std::atomic<long long> covered{0};
        parallel_for(L.num_blocks, 8, [&](int64_t b0, int64_t b1) {
            std::vector<int> cols, count;
            for (int64_t b = b0; b < b1; ++b) {
                const int e0 = rp[L.block_row[(size_t)b]], e1 = rp[L.block_row[(size_t)b + 1]];
                columns_in_order(e0, e1, cols, count);
                size_t best = 0, best_at = 0;
                for (size_t lo = 0, hi = 0; lo < cols.size(); ++lo) {
                    while (hi < cols.size() && cols[hi] < cols[lo] + W) ++hi;
                    if (hi - lo > best) {
                        best = hi - lo;
                        best_at = lo;
                    }
                }
                long long base = cols.empty() ? 0 : cols[best_at];
                base = std::max(0ll, std::min(base, (long long)n - W));  // all tables inside X where X has T H rows
                L.table_base[(size_t)b] = (int)base;
                covered.fetch_add((long long)best, std::memory_order_relaxed);
            }
        });
        if (!bp.local_tables && (double)covered.load() < bp.min_local_cover * (double)nnz) return kNotWorthwhile;
    }
    // Many short rows (fewer than 12 nonzeros per row, more than 2^18 rows): a window of the streams holds four
    // nonzeros of one row, step and kind, and the slab plans' sliced stream does as well on such rows - unless the
    // first table alone serves a good part of the nonzeros, or every block has one table of its own (block-diagonal,
    // 416,349 rows x 3 / 5 / 10: .023/.023, .025/.025, .029/.039 ms; 2,000,000 rows x 5: .103/.118; banded, 1,000,000
    // x 4 within 100 columns: .048/.055; but two tables per block, 2,000,000 x 8 within 500: .154/.138).
    if (!(local && T == 1) && bp.min_table_share_short_rows > 0.0 && n > (1 << 18) && (long long)nnz < 12LL * n &&
        (double)table_nnz[0] < bp.min_table_share_short_rows * (double)nnz)
        return kNotWorthwhile;
    if (bp.table_rows <= 0 && !local) {
        // no more slots than columns to put in them
        const int need = (n + T - 1) / T;
        if (H > need) H = need;
        H = (H + 3) / 4 * 4;
    }
    if (H < 1 || (long long)(H + L.acc_rows) * 64 + kSlotBytes > kLdsBytes) return MPS_ERR_INVALID_ARG;
    L.table_rows = H;
    L.steps = T;
    L.hot_bits = bits_for(H > 1 ? H - 1 : 1);
    const size_t R = std::min<size_t>((size_t)T * H, cand.size());
    if (!counted) {
        if (R < cand.size()) std::nth_element(cand.begin(), cand.begin() + (long)R, cand.end(), hotter);
        std::sort(cand.begin(), cand.begin() + (long)R, hotter);
    }
    cm.step.assign((size_t)n, 0);
    cm.slot.assign((size_t)n, -1);
    L.hot_cols.assign((size_t)T * H, -1);
    L.hot_nnz = 0;
    if (local) {
        cm.base = L.table_base.data();
        cm.H = H;
        cm.T = T;
        std::atomic<long long> in_tables{0};
        L.table_used.assign((size_t)L.num_blocks, 0);
        parallel_for(L.num_blocks, 1, [&](int64_t b0, int64_t b1) {
            long long hits = 0;
            for (int64_t b = b0; b < b1; ++b) {
                int used = 0;
                for (int e = rp[L.block_row[(size_t)b]]; e < rp[L.block_row[(size_t)b + 1]]; ++e) {
                    const int slot = cm.slot_of((int)b, ci[e]);
                    hits += slot >= 0;
                    if (slot >= 0 && cm.step_of((int)b, ci[e]) == T - 1) used = std::max(used, slot + 1);
                }
                L.table_used[(size_t)b] = used;
            }
            in_tables.fetch_add(hits, std::memory_order_relaxed);
        });
        L.hot_nnz = in_tables.load();
    }
    for (size_t k = 0; k < (local ? 0 : R); ++k) {
        const int c = cand[k];
        const int t = (int)(k % (size_t)T), slot = (int)(k / (size_t)T);
        cm.step[(size_t)c] = (int16_t)t;
        cm.slot[(size_t)c] = (int16_t)slot;
        L.hot_cols[(size_t)t * H + slot] = c;
        L.hot_nnz += d_of(c);
    }
    if (local) {
        L.cold_begin.assign((size_t)T + 1, 0);  // a block's cold columns lie anywhere outside its tables
        L.cold_begin[(size_t)T] = n;
    } else {
        const long long cold_total = (long long)nnz - L.hot_nnz;
        long long cum = 0;
        L.cold_begin.assign((size_t)T + 1, n);
        int t_prev = -1;
        for (int c = 0; c < n; ++c) {
            if (cm.slot[(size_t)c] >= 0) continue;
            int t = cold_total > 0 ? (int)std::min<long long>(T - 1, cum * T / cold_total) : 0;
            cm.step[(size_t)c] = (int16_t)t;
            for (int u = t_prev + 1; u <= t; ++u) L.cold_begin[(size_t)u] = c;
            t_prev = std::max(t_prev, t);
            cum += d_of(c);
        }
    }

    return MPS_OK;
}

// nonzeros per column
static void count_columns(const int *ci, int n, int nnz, std::vector<int> &deg)
{
    std::vector<std::atomic<int>> cnt((size_t)n);
    for (auto &d : cnt) d.store(0, std::memory_order_relaxed);
    parallel_for(nnz, 1 << 16, [&](int64_t a, int64_t b) {
        for (int64_t e = a; e < b; ++e) cnt[(size_t)ci[e]].fetch_add(1, std::memory_order_relaxed);
    });
    deg.resize((size_t)n);
    for (int c = 0; c < n; ++c) deg[(size_t)c] = cnt[(size_t)c].load(std::memory_order_relaxed);
}

int build_layout(const int *rp, const int *ci, const float *val, int n, int nnz, int K, const BuildParams &bp,
                 Layout &L)
{
    if (!rp || n < 1 || nnz < 0 || (nnz > 0 && (!ci || !val))) return MPS_ERR_INVALID_ARG;
    if (K != 16) return MPS_ERR_UNSUPPORTED;
    int H = 0;
    int rc = plan_blocks(rp, n, nnz, bp, L, &H);
    if (rc != MPS_OK) return rc;
    std::vector<int> deg;
    count_columns(ci, n, nnz, deg);
    // Share of the nonzeros in each block's busiest of R equal column ranges (own), and what the busiest range has
    // of the whole matrix.
    auto block_ranges = [&](int R, long long *own_out, long long *busiest_out) {
        std::vector<std::atomic<long long>> range_nnz((size_t)R);
        for (auto &c : range_nnz) c.store(0, std::memory_order_relaxed);
        std::atomic<long long> own{0};
        parallel_for(L.num_blocks, 1, [&](int64_t b0, int64_t b1) {
            std::vector<long long> cnt((size_t)R);
            for (int64_t b = b0; b < b1; ++b) {
                std::fill(cnt.begin(), cnt.end(), 0);
                for (int e = rp[L.block_row[(size_t)b]]; e < rp[L.block_row[(size_t)b + 1]]; ++e)
                    ++cnt[(size_t)((long long)ci[e] * R / n)];
                own.fetch_add(*std::max_element(cnt.begin(), cnt.end()), std::memory_order_relaxed);
                for (int r = 0; r < R; ++r) range_nnz[(size_t)r].fetch_add(cnt[(size_t)r], std::memory_order_relaxed);
            }
        });
        long long busiest = 0;
        for (auto &c : range_nnz) busiest = std::max(busiest, c.load(std::memory_order_relaxed));
        *own_out = own.load();
        *busiest_out = busiest;
    };
    ColumnMap cm;
    rc = plan_columns(rp, ci, n, nnz, bp, L, H, deg.data(), block_ranges, cm);
    if (rc != MPS_OK) return rc;
    const int T = L.steps;

    // ---- 4. pass 1: windows and first rows of every wavefront's runs
    const int NB = L.num_blocks;
    L.meta.assign((size_t)NB * T * kWaveSlots * 4, 0);
    std::vector<long long> rounds((size_t)NB * kWaveSlots * 2, 0);
    std::vector<int> cuts((size_t)NB * T * (kWaves + 1));  // where the runs of every (block, step) begin
    parallel_for(NB, 1, [&](int64_t b0, int64_t b1) {
        std::vector<int> cnt, before;
        for (int64_t b = b0; b < b1; ++b) {
            const int r0 = L.block_row[(size_t)b], nr = L.block_row[(size_t)b + 1] - r0;
            count_block(rp, ci, cm, (int)b, r0, nr, T, cnt);
            for (int t = 0; t < T; ++t) {
                StepSplit sp;
                split_step(cnt.data() + (size_t)t * nr * 2, nr, sp, before);
                std::copy(sp.cut, sp.cut + kWaves + 1, cuts.begin() + (ptrdiff_t)(((size_t)b * T + t) * (kWaves + 1)));
                for (int w = 0; w < kWaves; ++w) {
                    int *m = &L.meta[(((size_t)b * T + t) * kWaveSlots + w) * 4];
                    m[0] = sp.hstart[w + 1] - sp.hstart[w];
                    m[1] = sp.cstart[w + 1] - sp.cstart[w];
                    m[2] = sp.first_row[w];
                    rounds[((size_t)b * kWaveSlots + w) * 2 + 0] += rounds_for(m[0]);
                    rounds[((size_t)b * kWaveSlots + w) * 2 + 1] += rounds_for(m[1]);
                }
            }
        }
    });

    // ---- 5. where every wavefront's streams start
    L.wave_base.assign((size_t)NB * kWaveSlots * 2, 0);
    long long hr = 0, cr = 0;
    for (size_t i = 0; i < (size_t)NB * kWaveSlots; ++i) {
        L.wave_base[2 * i] = hr;
        L.wave_base[2 * i + 1] = cr;
        hr += rounds[2 * i];
        cr += rounds[2 * i + 1];
    }
    L.hot_rounds = hr;
    L.cold_rounds = cr;
    // (fresh vectors: what resize() hands out is zeroed memory only when it comes from the allocator)
    Zeroed<Entry>().swap(L.hot);
    Zeroed<Entry>().swap(L.cold);
    L.hot.resize((size_t)hr * kRoundEntries);
    L.cold.resize((size_t)cr * kRoundEntries);
    if (bp.keep_src) {
        L.hot_src.resize(L.hot.size());
        L.cold_src.resize(L.cold.size());
        for (std::vector<int> *v : {&L.hot_src, &L.cold_src})
            parallel_for((int64_t)v->size(), 1 << 16, [&](int64_t a, int64_t b) { std::fill(v->begin() + a, v->begin() + b, -1); });
    }

    // ---- 6. pass 2: place the entries
    parallel_for(NB, 1, [&](int64_t b0, int64_t b1) {
        std::vector<int> cnt, off, s_src;
        std::vector<uint32_t> s_idx;
        std::vector<float> s_val;
        for (int64_t b = b0; b < b1; ++b) {
            const int r0 = L.block_row[(size_t)b], nr = L.block_row[(size_t)b + 1] - r0;
            const int e0 = rp[r0], ne = rp[r0 + nr] - e0;
            count_block(rp, ci, cm, (int)b, r0, nr, T, cnt);
            off.resize(cnt.size() + 1);
            off[0] = 0;
            for (size_t i = 0; i < cnt.size(); ++i) off[i + 1] = off[i] + cnt[i];
            std::vector<int> t_begin((size_t)T + 1);
            for (int t = 0; t <= T; ++t) t_begin[(size_t)t] = off[(size_t)t * nr * 2];
            s_idx.resize((size_t)ne);
            s_val.resize((size_t)ne);
            s_src.resize((size_t)ne);
            for (int lr = 0; lr < nr; ++lr)
                for (int e = rp[r0 + lr]; e < rp[r0 + lr + 1]; ++e) {
                    const int c = ci[e];
                    const int slot = cm.slot_of((int)b, c);
                    const int k = slot < 0;
                    const int pos = off[((size_t)cm.step_of((int)b, c) * nr + lr) * 2 + k]++;
                    s_idx[(size_t)pos] = (uint32_t)(k ? c : slot);
                    s_val[(size_t)pos] = val[e];
                    s_src[(size_t)pos] = e;
                }
            long long round_off[kWaves][2];
            for (int w = 0; w < kWaves; ++w)
                for (int k = 0; k < 2; ++k) round_off[w][k] = L.wave_base[((size_t)b * kWaveSlots + w) * 2 + k];
            for (int t = 0; t < T; ++t) {
                const int *m0 = &L.meta[((size_t)b * T + t) * kWaveSlots * 4];
                const int *cnt_t = cnt.data() + (size_t)t * nr * 2;
                const int *cut = &cuts[((size_t)b * T + t) * (kWaves + 1)];
                int w = 0;
                long long w_end = cut[1];  // first window of run w + 1
                int placed[2] = {0, 0}, last_row[2] = {0, 0};
                long long q = 0;           // windows so far
                size_t p = (size_t)t_begin[(size_t)t];  // sorted nonzeros so far
                for (int lr = 0; lr < nr; ++lr)
                    for (int k = 0; k < 2; ++k) {
                        int left = cnt_t[2 * lr + k];
                        while (left > 0) {
                            while (q >= w_end) {
                                ++w;
                                w_end = cut[w + 1];
                                placed[0] = placed[1] = 0;
                            }
                            const int *m = m0 + w * 4;
                            int g, j;
                            deal(m[k], placed[k], &g, &j);
                            const int prev = j == 0 ? m[2] : last_row[k];
                            const uint32_t adv = (uint32_t)(lr - prev);
                            last_row[k] = lr;
                            ++placed[k];
                            // round j / 2; inside it lane (g, e) holds entry e of the group's two windows side by side
                            const size_t dst = (size_t)(round_off[w][k] + j / kPair) * kRoundEntries + (size_t)g * kWin * kPair + (size_t)(j % kPair);
                            const int take = left < kWin ? left : kWin;
                            Zeroed<Entry> &out = k ? L.cold : L.hot;
                            for (int e = 0; e < kWin; ++e) {
                                // padding repeats the window's last nonzero with value 0
                                const size_t src = p + (size_t)(e < take ? e : take - 1);
                                Entry en;
                                en.word = s_idx[src] | (e == 0 ? adv << (k ? L.cold_bits : L.hot_bits) : 0u);
                                en.val = e < take ? s_val[src] : 0.f;
                                out[dst + (size_t)e * kPair] = en;
                                if (bp.keep_src && e < take) (k ? L.cold_src : L.hot_src)[dst + (size_t)e * kPair] = s_src[src];
                            }
                            p += (size_t)take;
                            left -= take;
                            ++q;
                        }
                    }
                for (int ww = 0; ww < kWaves; ++ww)
                    for (int k = 0; k < 2; ++k) round_off[ww][k] += rounds_for(m0[ww * 4 + k]);
            }
        }
    });
    // what the device reads instead of L.hot (blocks hold at most 1,024 rows and tables at most 2,048: it always fits)
    if (!pack_hot_stream(L)) return MPS_ERR_UNSUPPORTED;
    pack_cold_stream(L);  // (or the device reads L.cold)
    return MPS_OK;
}

bool pack_hot_stream(Layout &L)
{
    L.hot_packed.clear();
    if (L.hot_bits > kPackedSlotBits) return false;
    const size_t rounds = L.hot.size() / kRoundEntries;
    const uint32_t slot_mask = (1u << L.hot_bits) - 1u, piece_mask = (1u << kPackedPieceBits) - 1u;
    std::atomic<bool> fits{true};
    Zeroed<uint32_t>().swap(L.hot_packed);
    L.hot_packed.resize(rounds * kPackedRoundWords);
    parallel_for((int64_t)rounds, 256, [&](int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; ++r)
            for (int lane = 0; lane < 64; ++lane) {
                // lane (g, e) holds entry e of its lane-group's two windows (A, B) side by side; entry 0 of a window
                // holds its rows_advanced, of which entry 0 keeps the low piece and entry 1 gets the high one
                const int e = lane % kWin, lane0 = lane - e;
                uint32_t halves[kPair];
                uint32_t *dst = &L.hot_packed[((size_t)r * 64 + (size_t)lane) * 3];
                for (int which = 0; which < kPair; ++which) {
                    const Entry &en = L.hot[(size_t)r * kRoundEntries + (size_t)lane * kPair + (size_t)which];
                    const uint32_t adv = L.hot[(size_t)r * kRoundEntries + (size_t)lane0 * kPair + (size_t)which].word >> L.hot_bits;
                    if (adv > kPackedAdvMax) fits.store(false, std::memory_order_relaxed);
                    const uint32_t piece = e == 0 ? (adv & piece_mask) : e == 1 ? ((adv >> kPackedPieceBits) & piece_mask) : 0u;
                    halves[which] = (en.word & slot_mask) | (piece << kPackedSlotBits);
                    std::memcpy(dst + which, &en.val, 4);
                }
                dst[2] = halves[0] | (halves[1] << 16);
            }
    });
    if (!fits.load()) L.hot_packed.clear();
    return fits.load();
}

bool pack_cold_stream(Layout &L)
{
    L.cold_packed.clear();
    L.cold_index_bits = 0;
    const int T = L.steps, NB = L.num_blocks;
    int widest = 1;
    for (int t = 0; t < T; ++t) widest = std::max(widest, L.cold_begin[(size_t)t + 1] - L.cold_begin[(size_t)t]);
    const int ib = std::max(12, bits_for(widest > 1 ? widest - 1 : 1));
    if (ib > 15) return false;
    const int pb = 16 - ib;
    const uint32_t idx_mask = (1u << L.cold_bits) - 1u, piece_mask = (1u << pb) - 1u;
    const uint32_t adv_max = pb * kWin >= 32 ? 0xffffffffu : (1u << (pb * kWin)) - 1u;
    std::atomic<bool> fits{true};
    Zeroed<uint32_t>().swap(L.cold_packed);
    L.cold_packed.resize((size_t)L.cold_rounds * kPackedRoundWords);
    parallel_for(NB, 1, [&](int64_t b0, int64_t b1) {
        for (int64_t b = b0; b < b1; ++b)
            for (int w = 0; w < kWaves; ++w) {
                long long r = L.wave_base[((size_t)b * kWaveSlots + (size_t)w) * 2 + 1];
                for (int t = 0; t < T; ++t) {
                    const int nc = L.meta[(((size_t)b * T + (size_t)t) * kWaveSlots + (size_t)w) * 4 + 1];
                    const int first = L.cold_begin[(size_t)t];
                    const int rounds = rounds_for(nc);
                    for (int q = 0; q < rounds; ++q, ++r)
                        for (int lane = 0; lane < 64; ++lane) {
                            const int g = lane / kWin, e = lane % kWin, lane0 = lane - e;
                            const int len = (nc >> 4) + (g < (nc & 15));  // windows of this lane-group in the run
                            uint32_t halves[kPair];
                            uint32_t *dst = &L.cold_packed[((size_t)r * 64 + (size_t)lane) * 3];
                            for (int which = 0; which < kPair; ++which) {
                                const Entry &en = L.cold[(size_t)r * kRoundEntries + (size_t)lane * kPair + (size_t)which];
                                std::memcpy(dst + which, &en.val, 4);
                                if (q * kPair + which >= len) {  // no window here: the gather still needs a row of X
                                    halves[which] = 0u;
                                    continue;
                                }
                                const uint32_t adv = L.cold[(size_t)r * kRoundEntries + (size_t)lane0 * kPair + (size_t)which].word >> L.cold_bits;
                                const int rel = (int)(en.word & idx_mask) - first;
                                if (adv > adv_max || rel < 0 || rel >= (1 << ib)) {
                                    fits.store(false, std::memory_order_relaxed);
                                    halves[which] = 0u;
                                    continue;
                                }
                                halves[which] = (uint32_t)rel | (((adv >> (pb * e)) & piece_mask) << ib);
                            }
                            dst[2] = halves[0] | (halves[1] << 16);
                        }
                }
            }
    });
    if (!fits.load()) {
        Zeroed<uint32_t>().swap(L.cold_packed);
        return false;
    }
    L.cold_index_bits = ib;
    return true;
}

}  // namespace mps_rb

struct mps_rowblock_layout {
    mps_rb::Layout L;
};

extern "C" {

int mps_rowblock_layout_build(const int *row_ptr, const int *col_idx, const float *val, int n_rows, int nnz, int K,
                              const mps_plan_options *options, mps_rowblock_layout **layout_out)
{
    if (!layout_out) return MPS_ERR_INVALID_ARG;
    *layout_out = nullptr;
    mps_rb::BuildParams bp;
    if (options) {
        bp.steps = options->rowblock_steps;
        bp.table_rows = options->rowblock_table_rows;
        bp.block_rows = options->rowblock_block_rows;
        bp.num_cus = options->rowblock_blocks_per_round;
        bp.keep_src = !(options->flags & MPS_PLAN_NO_SOURCES);
        bp.local_tables = (options->flags & MPS_PLAN_LOCAL_TABLES) != 0;
    }
    if (bp.num_cus <= 0) bp.num_cus = 256;
    mps_rowblock_layout *h = new (std::nothrow) mps_rowblock_layout;
    if (!h) return MPS_ERR_UNSUPPORTED;
    int rc;
    try {
        rc = mps_rb::build_layout(row_ptr, col_idx, val, n_rows, nnz, K, bp, h->L);
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

int mps_rowblock_layout_info(const mps_rowblock_layout *layout, mps_plan_info *info)
{
    if (!layout || !info) return MPS_ERR_INVALID_ARG;
    const mps_rb::Layout &L = layout->L;
    std::memset(info, 0, sizeof(*info));
    info->n_rows = L.n;
    info->nnz = L.nnz;
    info->K = L.K;
    info->elem_bytes = 4;
    info->num_slabs = 1;
    info->slab_cols = L.n;
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
    return MPS_OK;
}

int mps_rowblock_layout_array(const mps_rowblock_layout *layout, int which, const void **data_out, size_t *bytes_out)
{
    if (!layout || !data_out || !bytes_out) return MPS_ERR_INVALID_ARG;
    const mps_rb::Layout &L = layout->L;
    auto give = [&](const auto &v) {
        *data_out = v.data();
        *bytes_out = v.size() * sizeof(v[0]);
        return (int)MPS_OK;
    };
    switch (which) {
    case MPS_PLAN_ARRAY_RB_BLOCK_ROW: return give(L.block_row);
    case MPS_PLAN_ARRAY_RB_HOT_COLS: return give(L.hot_cols);
    case MPS_PLAN_ARRAY_RB_META: return give(L.meta);
    case MPS_PLAN_ARRAY_RB_WAVE_BASE: return give(L.wave_base);
    case MPS_PLAN_ARRAY_RB_HOT: return give(L.hot);
    case MPS_PLAN_ARRAY_RB_COLD: return give(L.cold);
    case MPS_PLAN_ARRAY_RB_HOT_SRC: return give(L.hot_src);
    case MPS_PLAN_ARRAY_RB_COLD_SRC: return give(L.cold_src);
    case MPS_PLAN_ARRAY_RB_HOT_PACKED: return give(L.hot_packed);
    case MPS_PLAN_ARRAY_RB_COLD_PACKED: return give(L.cold_packed);
    case MPS_PLAN_ARRAY_RB_COLD_BEGIN: return give(L.cold_begin);
    case MPS_PLAN_ARRAY_RB_TABLE_BASE: return give(L.table_base);
    default: return MPS_ERR_INVALID_ARG;
    }
}

void mps_rowblock_layout_free(mps_rowblock_layout *layout) { delete layout; }

}  // extern "C"
