// Host half of the MergePath-SpMM C ABI: status text, schedule arithmetic,
// .csr text I/O, seeded synthetic graphs and fills.  No GPU is touched here.
#include "mpspmm.h"
#include "mpspmm_internal.h"

#include <algorithm>
#include <atomic>
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <exception>
#include <map>
#include <mutex>
#include <string>
#include <system_error>
#include <thread>
#include <vector>

#include "mpspmm_hostpar.hpp"

namespace {

using mps_host::host_threads;
using mps_host::parallel_for;

// ---------------------------------------------------------------------------
// Counter-based random numbers (splitmix64 finaliser).
// ---------------------------------------------------------------------------
inline uint64_t mix64(uint64_t z)
{
    z += 0x9e3779b97f4a7c15ULL;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

struct Rng {
    uint64_t s;
    Rng(uint64_t seed, uint64_t stream) : s(mix64(mix64(seed) ^ (stream * 0xd1342543de82ef95ULL + 1))) {}
    uint64_t next()
    {
        s += 0x9e3779b97f4a7c15ULL;
        uint64_t z = s;
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
        return z ^ (z >> 31);
    }
    // uniform in (0, 1]
    double u01_open0() { return (double)((next() >> 11) + 1) * (1.0 / 9007199254740992.0); }
    // uniform in [0, 1)
    double u01() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
};

}  // namespace

struct mps_graph {
    std::vector<int> row_ptr;
    std::vector<int> col_idx;
    int max_degree = 0;
};

namespace {

void finish_graph(mps_graph *g)
{
    int n = (int)g->row_ptr.size() - 1;
    int md = 0;
    for (int i = 0; i < n; ++i) md = std::max(md, g->row_ptr[i + 1] - g->row_ptr[i]);
    g->max_degree = md;
}

// ---------------------------------------------------------------------------
// Spec strings: "name:key=value,key=value"
// ---------------------------------------------------------------------------
struct Spec {
    std::string name;
    std::map<std::string, double> kv;
    bool has(const char *k) const { return kv.count(k) != 0; }
    double get(const char *k, double dflt) const
    {
        auto it = kv.find(k);
        return it == kv.end() ? dflt : it->second;
    }
};

bool parse_spec(const char *text, Spec &out)
{
    std::string s(text);
    size_t colon = s.find(':');
    out.name = s.substr(0, colon);
    if (out.name.empty()) return false;
    if (colon == std::string::npos) return true;
    size_t pos = colon + 1;
    while (pos < s.size()) {
        size_t comma = s.find(',', pos);
        if (comma == std::string::npos) comma = s.size();
        std::string item = s.substr(pos, comma - pos);
        pos = comma + 1;
        if (item.empty()) continue;
        size_t eq = item.find('=');
        if (eq == std::string::npos || eq == 0) return false;
        char *end = nullptr;
        std::string v = item.substr(eq + 1);
        double d = std::strtod(v.c_str(), &end);
        if (end == v.c_str() || *end != '\0') return false;
        out.kv[item.substr(0, eq)] = d;
    }
    return true;
}

// Exclusive prefix sum of per-row counts into row_ptr; false on 32-bit overflow.
bool counts_to_row_ptr(const std::vector<int> &deg, std::vector<int> &row_ptr)
{
    size_t n = deg.size();
    row_ptr.resize(n + 1);
    int64_t run = 0;
    for (size_t i = 0; i < n; ++i) {
        row_ptr[i] = (int)run;
        run += deg[i];
        if (run > 0x7fffffffLL - (int64_t)n - 2) return false;
    }
    row_ptr[n] = (int)run;
    return true;
}

// ---------------------------------------------------------------------------
// Erdos-Renyi G(n, p = deg / n), directed, no self-loops.  Row i walks its
// columns with geometric skips drawn from its own stream.
// ---------------------------------------------------------------------------
template <typename Emit>
inline void er_row(uint64_t seed, int i, int n, double log1mp, Emit &&emit)
{
    Rng r(seed, (uint64_t)i);
    int64_t j = -1;
    for (;;) {
        double u = r.u01_open0();
        double skip = std::floor(std::log(u) / log1mp);
        if (skip > (double)n) break;
        j += 1 + (int64_t)skip;
        if (j >= n) break;
        if (j != i) emit((int)j);
    }
}

int gen_er(const Spec &sp, uint64_t seed, mps_graph *g)
{
    int n = (int)sp.get("n", 4096);
    double deg = sp.get("deg", 8);
    if (n < 2 || deg <= 0 || deg >= n) return MPS_ERR_FORMAT;
    double p = deg / (double)n;
    double log1mp = std::log1p(-p);
    std::vector<int> cnt(n);
    parallel_for(n, 1024, [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i) {
            int c = 0;
            er_row(seed, (int)i, n, log1mp, [&](int) { ++c; });
            cnt[i] = c;
        }
    });
    if (!counts_to_row_ptr(cnt, g->row_ptr)) return MPS_ERR_UNSUPPORTED;
    g->col_idx.resize(g->row_ptr[n]);
    parallel_for(n, 1024, [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i) {
            int *dst = g->col_idx.data() + g->row_ptr[i];
            er_row(seed, (int)i, n, log1mp, [&](int j) { *dst++ = j; });
        }
    });
    return MPS_OK;
}

// ---------------------------------------------------------------------------
// Banded: column j of row i present independently with probability
// deg / (2 width + 1) for 0 < |i - j| <= width (Erdos-Renyi inside the band,
// no self-loops; rows near the ends are shorter).
// ---------------------------------------------------------------------------
template <typename Emit>
inline void band_row(uint64_t seed, int i, int n, int width, double log1mp, Emit &&emit)
{
    Rng r(seed, (uint64_t)i);
    const int64_t first = std::max<int64_t>(0, (int64_t)i - width), last = std::min<int64_t>(n - 1, (int64_t)i + width);
    int64_t j = first - 1;
    for (;;) {
        double u = r.u01_open0();
        double skip = std::floor(std::log(u) / log1mp);
        if (skip > (double)(2 * (int64_t)width + 1)) break;
        j += 1 + (int64_t)skip;
        if (j > last) break;
        if (j != i) emit((int)j);
    }
}

int gen_band(const Spec &sp, uint64_t seed, mps_graph *g)
{
    int n = (int)sp.get("n", 4096);
    double deg = sp.get("deg", 8);
    int width = (int)sp.get("width", 64);
    if (n < 2 || width < 1 || width >= n || deg <= 0 || deg >= 2.0 * width + 1) return MPS_ERR_FORMAT;
    double log1mp = std::log1p(-deg / (2.0 * width + 1));
    std::vector<int> cnt(n);
    parallel_for(n, 1024, [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i) {
            int c = 0;
            band_row(seed, (int)i, n, width, log1mp, [&](int) { ++c; });
            cnt[i] = c;
        }
    });
    if (!counts_to_row_ptr(cnt, g->row_ptr)) return MPS_ERR_UNSUPPORTED;
    g->col_idx.resize(g->row_ptr[n]);
    parallel_for(n, 1024, [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i) {
            int *dst = g->col_idx.data() + g->row_ptr[i];
            band_row(seed, (int)i, n, width, log1mp, [&](int j) { *dst++ = j; });
        }
    });
    return MPS_OK;
}

// ---------------------------------------------------------------------------
// Chung-Lu: edge (u, v), u != v, present independently with probability
// min(1, w_u w_v / S).  Expected degrees follow a shifted power law over the
// rank r = 0..n-1:  w_r = dmax * (1 + r / r0)^(-1 / (gamma - 1)); r0 is
// solved so that the expected number of edges equals the requested nnz.
// Each row walks the ranks with the skipping method of Miller & Hagberg
// (weights are non-increasing in rank, so the acceptance ratio is <= 1).
// Ranks are then relabelled by a seeded random permutation (unless
// sorted=1), and every row's columns sorted.
// ---------------------------------------------------------------------------
struct ChungLu {
    int n;
    std::vector<double> w;
    double S;
};

double chunglu_expected_edges(const ChungLu &c, const std::vector<double> &prefix)
{
    // sum_u sum_{v != u} min(1, w_u w_v / S); w non-increasing.
    double total = 0;
    int n = c.n;
    int vstar = n;  // first v with w_u * w_v < S  (decreases... grows as u grows)
    // For u ascending w_u decreases, so the saturated prefix [0, v*) shrinks.
    vstar = n;
    for (int u = 0; u < n; ++u) {
        double wu = c.w[u];
        // largest count of leading v with wu * w_v >= S
        while (vstar > 0 && wu * c.w[vstar - 1] < c.S) --vstar;
        double sat = vstar;
        double rest = (prefix[n] - prefix[vstar]) * wu / c.S;
        double self = (u < vstar) ? 1.0 : wu * wu / c.S;
        total += sat + rest - self;
    }
    return total;
}

void chunglu_weights(ChungLu &c, double dmax, double alpha, double r0, std::vector<double> &prefix)
{
    int n = c.n;
    c.w.resize(n);
    prefix.resize(n + 1);
    prefix[0] = 0;
    for (int r = 0; r < n; ++r) {
        c.w[r] = dmax * std::pow(1.0 + (double)r / r0, -alpha);
        prefix[r + 1] = prefix[r] + c.w[r];
    }
    c.S = prefix[n];
}

template <typename Emit>
inline void chunglu_row(const ChungLu &c, uint64_t seed, int u, Emit &&emit)
{
    Rng r(seed, (uint64_t)u);
    const int n = c.n;
    const double wu_over_S = c.w[u] / c.S;
    int64_t v = 0;
    double p = std::min(1.0, wu_over_S * c.w[0]);
    while (v < n && p > 0) {
        if (p < 1.0) {
            double x = r.u01_open0();
            double skip = std::floor(std::log(x) / std::log1p(-p));
            if (skip > (double)n) break;
            v += (int64_t)skip;
        }
        if (v < n) {
            double q = std::min(1.0, wu_over_S * c.w[v]);
            if (r.u01() < q / p) {
                if ((int)v != u) emit((int)v);
            }
            p = q;
            ++v;
        }
    }
}

int gen_chunglu(const Spec &sp, uint64_t seed, mps_graph *g)
{
    int n = (int)sp.get("n", 232965);
    double target = sp.get("nnz", 114.6e6);
    double gamma = sp.get("gamma", 2.1);
    double dmax = sp.get("dmax", 20000);
    bool sorted_labels = sp.get("sorted", 0) != 0;
    if (n < 2 || gamma <= 1.0 || dmax <= 0 || target <= 0) return MPS_ERR_FORMAT;
    if (target > 2.0e9 || target >= (double)n * (n - 1)) return MPS_ERR_UNSUPPORTED;
    if (dmax > n - 1) dmax = n - 1;
    double alpha = 1.0 / (gamma - 1.0);

    ChungLu c;
    c.n = n;
    std::vector<double> prefix;
    // Bisection on log(r0): expected edges grow with r0 (flatter weights).
    double lo = std::log(1e-6), hi = std::log(1e12);
    for (int it = 0; it < 80; ++it) {
        double mid = 0.5 * (lo + hi);
        chunglu_weights(c, dmax, alpha, std::exp(mid), prefix);
        if (chunglu_expected_edges(c, prefix) < target) lo = mid; else hi = mid;
    }
    chunglu_weights(c, dmax, alpha, std::exp(0.5 * (lo + hi)), prefix);

    // rank -> label
    std::vector<int> label(n);
    for (int i = 0; i < n; ++i) label[i] = i;
    if (!sorted_labels) {
        Rng pr(seed, 0xC0FFEEULL << 20);
        for (int i = n - 1; i > 0; --i) {
            int j = (int)(pr.next() % (uint64_t)(i + 1));
            std::swap(label[i], label[j]);
        }
    }

    // Pass 1: rows in rank space, kept per chunk of ranks.
    const int grain = 256;
    int chunks = (n + grain - 1) / grain;
    std::vector<std::vector<int>> chunk_cols(chunks);
    std::vector<int> deg_rank(n), deg_label(n);
    parallel_for(n, grain, [&](int64_t lo_r, int64_t hi_r) {
        std::vector<int> &buf = chunk_cols[lo_r / grain];
        for (int64_t u = lo_r; u < hi_r; ++u) {
            size_t before = buf.size();
            chunglu_row(c, seed, (int)u, [&](int v) { buf.push_back(v); });
            deg_rank[u] = (int)(buf.size() - before);
        }
    });
    for (int u = 0; u < n; ++u) deg_label[label[u]] = deg_rank[u];
    if (!counts_to_row_ptr(deg_label, g->row_ptr)) return MPS_ERR_UNSUPPORTED;
    g->col_idx.resize(g->row_ptr[n]);
    // Pass 2: relabel, place, sort.
    parallel_for(n, grain, [&](int64_t lo_r, int64_t hi_r) {
        const std::vector<int> &buf = chunk_cols[lo_r / grain];
        size_t off = 0;
        for (int64_t u = lo_r; u < hi_r; ++u) {
            int *dst = g->col_idx.data() + g->row_ptr[label[u]];
            int d = deg_rank[u];
            for (int k = 0; k < d; ++k) dst[k] = label[buf[off + k]];
            off += d;
            if (!sorted_labels) std::sort(dst, dst + d);
        }
    });
    return MPS_OK;
}

// ---------------------------------------------------------------------------
// Block-diagonal random-geometric graph: `blocks` disjoint blocks with sizes
// uniform in [min, max]; inside a block, points uniform in the unit square,
// an (undirected) edge between points closer than r, with r solved so that
// the expected degree is `deg` (exact distance distribution in the square).
// ---------------------------------------------------------------------------
double rgg_radius(int n, double deg)
{
    if (n < 2) return 0;
    double target = deg / (double)(n - 1);
    if (target >= 0.97) return 1.0;
    double lo = 0, hi = 1.0;
    for (int it = 0; it < 60; ++it) {
        double r = 0.5 * (lo + hi);
        double p = M_PI * r * r - 8.0 / 3.0 * r * r * r + 0.5 * r * r * r * r;
        if (p < target) lo = r; else hi = r;
    }
    return 0.5 * (lo + hi);
}

int gen_blockdiag(const Spec &sp, uint64_t seed, mps_graph *g)
{
    int blocks = (int)sp.get("blocks", 1178);
    int bmin = (int)sp.get("min", 100), bmax = (int)sp.get("max", 600);
    double deg = sp.get("deg", 5);
    if (blocks < 1 || bmin < 2 || bmax < bmin || deg <= 0) return MPS_ERR_FORMAT;
    std::vector<int> bstart(blocks + 1);
    {
        Rng r(seed, 0xB10CULL << 24);
        int64_t run = 0;
        for (int b = 0; b < blocks; ++b) {
            bstart[b] = (int)run;
            run += bmin + (int)(r.next() % (uint64_t)(bmax - bmin + 1));
            if (run > 0x3fffffff) return MPS_ERR_UNSUPPORTED;
        }
        bstart[blocks] = (int)run;
    }
    int n = bstart[blocks];
    std::vector<int> cnt(n);
    std::vector<float> px(n), py(n);
    parallel_for(blocks, 1, [&](int64_t lo, int64_t hi) {
        for (int64_t b = lo; b < hi; ++b) {
            Rng r(seed, (uint64_t)b + 1);
            for (int i = bstart[b]; i < bstart[b + 1]; ++i) {
                px[i] = (float)r.u01();
                py[i] = (float)r.u01();
            }
        }
    });
    auto block_rows = [&](int64_t b, bool fill) {
        int s = bstart[b], e = bstart[b + 1];
        double rr = rgg_radius(e - s, deg);
        float r2 = (float)(rr * rr);
        for (int i = s; i < e; ++i) {
            int c = 0;
            int *dst = fill ? g->col_idx.data() + g->row_ptr[i] : nullptr;
            for (int j = s; j < e; ++j) {
                if (j == i) continue;
                float dx = px[i] - px[j], dy = py[i] - py[j];
                if (dx * dx + dy * dy <= r2) {
                    if (fill) dst[c] = j;
                    ++c;
                }
            }
            if (!fill) cnt[i] = c;
        }
    };
    parallel_for(blocks, 1, [&](int64_t lo, int64_t hi) {
        for (int64_t b = lo; b < hi; ++b) block_rows(b, false);
    });
    if (!counts_to_row_ptr(cnt, g->row_ptr)) return MPS_ERR_UNSUPPORTED;
    g->col_idx.resize(g->row_ptr[n]);
    parallel_for(blocks, 1, [&](int64_t lo, int64_t hi) {
        for (int64_t b = lo; b < hi; ++b) block_rows(b, true);
    });
    return MPS_OK;
}

// ---------------------------------------------------------------------------
// R-MAT: ef * 2^scale directed edges, each placed by `scale` recursive
// quadrant choices with probabilities (a, b, c, 1-a-b-c); duplicate edges are
// removed, self-loops kept.  Edge e draws from its own stream.
// ---------------------------------------------------------------------------
inline void rmat_edge(uint64_t seed, uint64_t e, int scale, uint32_t ta, uint32_t tab, uint32_t tabc,
                      int &src, int &dst)
{
    Rng r(seed, e);
    uint32_t s = 0, d = 0;
    uint64_t bits = 0;
    int have = 0;
    for (int l = 0; l < scale; ++l) {
        if (have == 0) {
            bits = r.next();
            have = 4;
        }
        uint32_t u = (uint32_t)(bits & 0xffff);
        bits >>= 16;
        --have;
        s <<= 1;
        d <<= 1;
        if (u < ta) {
        } else if (u < tab) {
            d |= 1;
        } else if (u < tabc) {
            s |= 1;
        } else {
            s |= 1;
            d |= 1;
        }
    }
    src = (int)s;
    dst = (int)d;
}

int gen_rmat(const Spec &sp, uint64_t seed, mps_graph *g)
{
    int scale = (int)sp.get("scale", 20);
    double ef = sp.get("ef", 16);
    double a = sp.get("a", 0.57), b = sp.get("b", 0.19), c = sp.get("c", 0.19);
    if (scale < 1 || scale > 26 || ef <= 0 || a <= 0 || b < 0 || c < 0 || a + b + c >= 1.0)
        return MPS_ERR_FORMAT;
    int n = 1 << scale;
    double m_d = ef * (double)n;
    if (m_d > 2.0e9) return MPS_ERR_UNSUPPORTED;
    int64_t m = (int64_t)m_d;
    uint32_t ta = (uint32_t)std::lround(a * 65536.0);
    uint32_t tab = (uint32_t)std::lround((a + b) * 65536.0);
    uint32_t tabc = (uint32_t)std::lround((a + b + c) * 65536.0);

    std::vector<std::atomic<int>> cursor(n);
    for (int i = 0; i < n; ++i) cursor[i].store(0, std::memory_order_relaxed);
    parallel_for(m, 1 << 16, [&](int64_t lo, int64_t hi) {
        for (int64_t e = lo; e < hi; ++e) {
            int s, d;
            rmat_edge(seed, (uint64_t)e, scale, ta, tab, tabc, s, d);
            cursor[s].fetch_add(1, std::memory_order_relaxed);
        }
    });
    std::vector<int> cnt(n);
    for (int i = 0; i < n; ++i) cnt[i] = cursor[i].load(std::memory_order_relaxed);
    std::vector<int> rp0;
    if (!counts_to_row_ptr(cnt, rp0)) return MPS_ERR_UNSUPPORTED;
    std::vector<int> cols0(rp0[n]);
    for (int i = 0; i < n; ++i) cursor[i].store(rp0[i], std::memory_order_relaxed);
    parallel_for(m, 1 << 16, [&](int64_t lo, int64_t hi) {
        for (int64_t e = lo; e < hi; ++e) {
            int s, d;
            rmat_edge(seed, (uint64_t)e, scale, ta, tab, tabc, s, d);
            int pos = cursor[s].fetch_add(1, std::memory_order_relaxed);
            cols0[pos] = d;
        }
    });
    // sort + unique every row (placement order above is not deterministic, the
    // sorted distinct set is)
    parallel_for(n, 512, [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i) {
            int *b0 = cols0.data() + rp0[i], *e0 = cols0.data() + rp0[i + 1];
            std::sort(b0, e0);
            cnt[i] = (int)(std::unique(b0, e0) - b0);
        }
    });
    if (!counts_to_row_ptr(cnt, g->row_ptr)) return MPS_ERR_UNSUPPORTED;
    g->col_idx.resize(g->row_ptr[n]);
    parallel_for(n, 512, [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i)
            std::copy(cols0.data() + rp0[i], cols0.data() + rp0[i] + cnt[i],
                      g->col_idx.data() + g->row_ptr[i]);
    });
    return MPS_OK;
}

// ---------------------------------------------------------------------------
// .csr text
// ---------------------------------------------------------------------------
bool read_whole_file(const char *path, std::vector<char> &buf)
{
    FILE *f = std::fopen(path, "rb");
    if (!f) return false;
    if (std::fseek(f, 0, SEEK_END) != 0) { std::fclose(f); return false; }
    long sz = std::ftell(f);
    if (sz < 0) { std::fclose(f); return false; }
    std::rewind(f);
    buf.resize((size_t)sz);
    size_t got = sz ? std::fread(buf.data(), 1, (size_t)sz, f) : 0;
    std::fclose(f);
    return got == (size_t)sz;
}

// Parses one line of comma-separated integers starting at p (stops at '\n' or
// end).  Cells are separated by ','; a ',' directly before the line end adds
// no cell; blanks around a number are skipped.  Returns the number of cells,
// or -1 on a malformed cell.  If out != nullptr at most cap values are stored.
int64_t parse_line(const char *&p, const char *end, int *out, int64_t cap, int *last)
{
    int64_t count = 0;
    while (p < end && *p != '\n') {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
        if (p >= end || *p == '\n') break;
        bool neg = false;
        if (*p == '-' || *p == '+') { neg = (*p == '-'); ++p; }
        if (p >= end || *p < '0' || *p > '9') return -1;
        int64_t v = 0;
        while (p < end && *p >= '0' && *p <= '9') {
            v = v * 10 + (*p - '0');
            if (v > 0x7fffffffLL) return -1;
            ++p;
        }
        if (neg) v = -v;
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
        if (p < end && *p == ',') ++p;
        else if (p < end && *p != '\n') return -1;
        if (out && count < cap) out[count] = (int)v;
        if (last) *last = (int)v;
        ++count;
    }
    if (p < end && *p == '\n') ++p;
    return count;
}

// One line of the file, [b, e) without the newline, cut at commas into pieces
// that are parsed side by side: a counting pass gives every piece its place in
// the output, a second pass stores the cells.  Returns the number of cells, or
// -1 on a malformed cell; at most cap values are stored.
int64_t parse_line_parallel(const char *b, const char *e, int *out, int64_t cap)
{
    const int64_t bytes = e - b;
    const int64_t piece = 1 << 20;
    if (bytes <= 2 * piece || host_threads() <= 1) {
        const char *p = b;
        return parse_line(p, e, out, cap, nullptr);
    }
    const int64_t pieces = (bytes + piece - 1) / piece;
    std::vector<const char *> cut((size_t)pieces + 1);
    cut[0] = b;
    cut[(size_t)pieces] = e;
    for (int64_t i = 1; i < pieces; ++i) {  // a piece starts right behind a comma
        const char *p = b + i * piece;
        while (p < e && p[-1] != ',') ++p;
        cut[(size_t)i] = p;
    }
    std::vector<int64_t> cells((size_t)pieces + 1, 0);
    std::atomic<bool> bad(false);
    parallel_for(pieces, 1, [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i) {
            const char *p = cut[(size_t)i];
            int64_t c = parse_line(p, cut[(size_t)i + 1], nullptr, 0, nullptr);
            if (c < 0) bad = true;
            cells[(size_t)i + 1] = c < 0 ? 0 : c;
        }
    });
    if (bad) return -1;
    for (int64_t i = 0; i < pieces; ++i) cells[(size_t)i + 1] += cells[(size_t)i];
    if (out) {
        parallel_for(pieces, 1, [&](int64_t lo, int64_t hi) {
            for (int64_t i = lo; i < hi; ++i) {
                const int64_t at = cells[(size_t)i];
                if (at >= cap) continue;
                const char *p = cut[(size_t)i];
                parse_line(p, cut[(size_t)i + 1], out + at, cap - at, nullptr);
            }
        });
    }
    return cells[(size_t)pieces];
}

int parse_csr(const std::vector<char> &buf, int n_rows, int nnz, int *row_ptr, int *col_idx)
{
    const char *b = buf.data(), *end = buf.data() + buf.size();
    const char *nl = static_cast<const char *>(std::memchr(b, '\n', buf.size()));
    const char *e1 = nl ? nl : end;
    int64_t c1 = parse_line_parallel(b, e1, row_ptr, (int64_t)n_rows + 1);
    if (c1 != (int64_t)n_rows + 1) return MPS_ERR_FORMAT;
    const char *b2 = nl ? nl + 1 : end;
    const char *nl2 = b2 < end ? static_cast<const char *>(std::memchr(b2, '\n', (size_t)(end - b2))) : nullptr;
    int64_t c2 = parse_line_parallel(b2, nl2 ? nl2 : end, col_idx, nnz);
    if (c2 != nnz) return MPS_ERR_FORMAT;
    if (row_ptr[0] != 0 || row_ptr[n_rows] != nnz) return MPS_ERR_FORMAT;
    std::atomic<bool> bad(false);
    parallel_for(n_rows, 1 << 16, [&](int64_t lo, int64_t hi) {
        for (int64_t i = lo; i < hi; ++i)
            if (row_ptr[i + 1] < row_ptr[i]) bad = true;
    });
    parallel_for(nnz, 1 << 18, [&](int64_t lo, int64_t hi) {
        for (int64_t k = lo; k < hi; ++k)
            if (col_idx[k] < 0 || col_idx[k] >= n_rows) bad = true;
    });
    return bad ? MPS_ERR_FORMAT : MPS_OK;
}

int header_from_buf(const std::vector<char> &buf, int *n_rows, int *nnz)
{
    const char *b = buf.data(), *end = buf.data() + buf.size();
    const char *nl = static_cast<const char *>(std::memchr(b, '\n', buf.size()));
    const char *e1 = nl ? nl : end;
    int64_t cells = parse_line_parallel(b, e1, nullptr, 0);
    // the last cell of the line is nnz (src/MergePathSpMM.cu:131-137)
    int last = 0;
    {
        const char *q = e1;
        while (q > b && (q[-1] == ',' || q[-1] == ' ' || q[-1] == '\t' || q[-1] == '\r')) --q;
        const char *t = q;
        while (t > b && t[-1] != ',') --t;
        const char *p = t;
        if (cells >= 1 && parse_line(p, q, nullptr, 0, &last) != 1) return MPS_ERR_FORMAT;
    }
    if (cells < 1 || cells > 0x7fffffffLL || last < 0) return MPS_ERR_FORMAT;
    if ((int64_t)cells + last > 0x7fffffffLL) return MPS_ERR_UNSUPPORTED;
    *n_rows = (int)cells - 1;
    *nnz = last;
    return MPS_OK;
}

inline uint16_t float_to_half_bits(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    int32_t exp = (int32_t)((x >> 23) & 0xff) - 127 + 15;
    uint32_t man = x & 0x7fffffu;
    if (((x >> 23) & 0xff) == 0xff) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0));
    if (exp >= 31) return (uint16_t)(sign | 0x7c00u);
    if (exp <= 0) {
        if (exp < -10) return (uint16_t)sign;
        man |= 0x800000u;
        int shift = 14 - exp;
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) ++half_man;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = sign | ((uint32_t)exp << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) ++half;
    return (uint16_t)half;
}

}  // namespace

// ===========================================================================
// C ABI
// ===========================================================================
extern "C" {

const char *mps_status_string(int status)
{
    switch (status) {
    case MPS_OK: return "ok";
    case MPS_ERR_INVALID_ARG: return "invalid argument";
    case MPS_ERR_UNSUPPORTED: return "unsupported size or shape";
    case MPS_ERR_WORKSPACE: return "workspace missing or too small";
    case MPS_ERR_ALIGNMENT: return "device pointer not sufficiently aligned";
    case MPS_ERR_IO: return "file cannot be opened, read or written";
    case MPS_ERR_FORMAT: return "malformed .csr text or generator spec";
    case MPS_ERR_TPW: return "threads_per_wave exceeds what one wavefront holds";
    case MPS_ERR_INVALID_CSR: return "CSR arrays failed validation";
    case MPS_ERR_UNSORTED: return "column ids are not sorted within every row";
    default: break;
    }
    if (status >= MPS_ERR_HIP) return "HIP runtime error (status - 1000 is the hipError_t)";
    return "unknown status";
}

const char *mps_version(void) { return "0.1.0"; }

int mps_num_partitions(int n_rows, int nnz, int cost, int *P_out)
{
    if (!P_out || n_rows < 0 || nnz < 0 || cost <= 0) return MPS_ERR_INVALID_ARG;
    if ((int64_t)n_rows + 1 + nnz > 0x7fffffffLL) return MPS_ERR_UNSUPPORTED;
    int node_act_num = n_rows + 1;
    int P = (node_act_num + nnz - 1) / cost;
    if (P < 1024) P = 1024;
    *P_out = P;
    return MPS_OK;
}

int mps_default_cost(int n_rows, int nnz, int K, int elem_bytes, int *cost_out)
{
    if (!cost_out || n_rows < 0 || nnz < 0 || K <= 0 || (elem_bytes != 2 && elem_bytes != 4)) return MPS_ERR_INVALID_ARG;
    const int64_t total = (int64_t)n_rows + 1 + nnz;
    const int by_size = total >= (1 << 27) ? 128 : total >= (1 << 25) ? 64 : 32;
    // A wavefront should have some 512 merge items whatever number of partitions it holds,
    // twice that where rows are long (32 nonzeros and more on average).  Measured on MI355X:
    // R-MAT graphs (15 per row) run best at 512 items per wavefront for every K (scale 22, fp16,
    // K = 64: cost 64 1.23 ms, 128 1.27 ms, 256 1.33 ms); the 232,965-row power-law graph (492
    // per row) at 1,024 or more (K = 32 fp32: cost 64 0.99 ms, 128 0.93 ms; fp16 K = 64: cost 64
    // 1.10 ms, 128 0.99 ms), K = 16 fp32 at its 16 x 64 either way.
    const int groups = mps_make_lane_shape(K, elem_bytes).groups;
    const bool long_rows = n_rows > 0 && (int64_t)nnz >= 32 * (int64_t)n_rows;
    const int by_width = (long_rows ? 1024 : 512) / groups;  // 32 (16 groups, short rows) .. 1024 (one group, long rows)
    *cost_out = by_size > by_width ? by_size : by_width;
    return MPS_OK;
}

int mps_items_per_partition(int n_rows, int nnz, int P, int *ipt_out)
{
    if (!ipt_out || n_rows < 0 || nnz < 0 || P <= 0) return MPS_ERR_INVALID_ARG;
    int64_t total = (int64_t)n_rows + 1 + nnz;
    if (total > 0x7fffffffLL) return MPS_ERR_UNSUPPORTED;
    *ipt_out = (int)((total + P - 1) / P);
    return MPS_OK;
}

int mps_partition_host(const int *row_ptr, int n_rows, int nnz, int P, int *coord_x, int *coord_y)
{
    if (!row_ptr || !coord_x || !coord_y || n_rows < 0 || nnz < 0 || P < 1) return MPS_ERR_INVALID_ARG;
    int ipt = 0;
    int rc = mps_items_per_partition(n_rows, nnz, P, &ipt);
    if (rc != MPS_OK) return rc;
    const int num_rows = n_rows + 1;  // the search runs over all of row_ptr, row_ptr[0] included (:333-334)
    const int64_t total = (int64_t)num_rows + nnz;
    parallel_for((int64_t)P + 1, 4096, [&](int64_t a, int64_t b) {
        for (int64_t i = a; i < b; ++i) {
            const int64_t d64 = (int64_t)ipt * i;
            const int diagonal = (int)(d64 < total ? d64 : total);
            // smallest x with row_ptr[x] + x >= diagonal: what the bisection of :283-295 finds
            int lo = diagonal > nnz ? diagonal - nnz : 0, hi = diagonal < num_rows ? diagonal : num_rows;
            while (lo < hi) {
                const int mid = (int)(((int64_t)lo + hi) >> 1);
                if (row_ptr[mid] <= diagonal - mid - 1) lo = mid + 1; else hi = mid;
            }
            coord_x[i] = lo < num_rows ? lo : num_rows;
            coord_y[i] = diagonal - lo;
        }
    });
    return MPS_OK;
}

int mps_max_threads_per_wave(int K, int elem_bytes, int *tpw_out)
{
    if (!tpw_out || K < 1 || (elem_bytes != 4 && elem_bytes != 2)) return MPS_ERR_INVALID_ARG;
    *tpw_out = mps_make_lane_shape(K, elem_bytes).groups;
    return MPS_OK;
}

int mps_csr_read_header(const char *path, int *n_rows_out, int *nnz_out)
{
    if (!path || !n_rows_out || !nnz_out) return MPS_ERR_INVALID_ARG;
    try {
        std::vector<char> buf;
        if (!read_whole_file(path, buf)) return MPS_ERR_IO;
        return header_from_buf(buf, n_rows_out, nnz_out);
    } catch (const std::bad_alloc &) {
        return MPS_ERR_UNSUPPORTED;
    }
}

int mps_csr_read(const char *path, int n_rows, int nnz, int *row_ptr, int *col_idx)
{
    if (!path || !row_ptr || (!col_idx && nnz > 0) || n_rows < 0 || nnz < 0) return MPS_ERR_INVALID_ARG;
    try {
        std::vector<char> buf;
        if (!read_whole_file(path, buf)) return MPS_ERR_IO;
        return parse_csr(buf, n_rows, nnz, row_ptr, col_idx);
    } catch (const std::bad_alloc &) {
        return MPS_ERR_UNSUPPORTED;
    }
}

int mps_csr_write(const char *path, int n_rows, const int *row_ptr, const int *col_idx)
{
    if (!path || !row_ptr || n_rows < 0) return MPS_ERR_INVALID_ARG;
    int nnz = row_ptr[n_rows];
    if (nnz < 0 || (nnz > 0 && !col_idx)) return MPS_ERR_INVALID_ARG;
    FILE *f = std::fopen(path, "wb");
    if (!f) return MPS_ERR_IO;
    std::vector<char> out;
    out.reserve(1 << 20);
    auto flush = [&]() -> bool {
        bool ok = out.empty() || std::fwrite(out.data(), 1, out.size(), f) == out.size();
        out.clear();
        return ok;
    };
    auto put = [&](int v) {
        char tmp[16];
        int len = std::snprintf(tmp, sizeof tmp, "%d,", v);
        out.insert(out.end(), tmp, tmp + len);
    };
    bool ok = true;
    for (int i = 0; i <= n_rows && ok; ++i) {
        put(row_ptr[i]);
        if (out.size() > (1 << 20) - 32) ok = flush();
    }
    out.push_back('\n');
    for (int e = 0; e < nnz && ok; ++e) {
        put(col_idx[e]);
        if (out.size() > (1 << 20) - 32) ok = flush();
    }
    ok = ok && flush();
    ok = (std::fclose(f) == 0) && ok;
    return ok ? MPS_OK : MPS_ERR_IO;
}

int mps_graph_generate(const char *spec, uint64_t seed, mps_graph **graph_out)
{
    if (!spec || !graph_out) return MPS_ERR_INVALID_ARG;
    *graph_out = nullptr;
    Spec sp;
    if (!parse_spec(spec, sp)) return MPS_ERR_FORMAT;
    mps_graph *g = new (std::nothrow) mps_graph;
    if (!g) return MPS_ERR_UNSUPPORTED;
    int rc;
    try {
        if (sp.name == "er") rc = gen_er(sp, seed, g);
        else if (sp.name == "chunglu") rc = gen_chunglu(sp, seed, g);
        else if (sp.name == "blockdiag") rc = gen_blockdiag(sp, seed, g);
        else if (sp.name == "rmat") rc = gen_rmat(sp, seed, g);
        else if (sp.name == "band") rc = gen_band(sp, seed, g);
        else rc = MPS_ERR_FORMAT;
    } catch (const std::bad_alloc &) {
        rc = MPS_ERR_UNSUPPORTED;
    }
    if (rc != MPS_OK) {
        delete g;
        return rc;
    }
    finish_graph(g);
    *graph_out = g;
    return MPS_OK;
}

int mps_graph_from_edges(const int64_t *src, const int64_t *dst, int64_t n_edges, mps_graph **graph_out)
{
    if (!graph_out || n_edges < 0 || (n_edges > 0 && (!src || !dst))) return MPS_ERR_INVALID_ARG;
    *graph_out = nullptr;
    int64_t top = -1;
    for (int64_t e = 0; e < n_edges; ++e) {
        if (src[e] < 0 || dst[e] < 0) return MPS_ERR_FORMAT;
        top = std::max(top, std::max(src[e], dst[e]));
    }
    const int64_t n64 = top + 1;
    if (n64 + 1 + n_edges > 0x7fffffffLL) return MPS_ERR_UNSUPPORTED;
    const int n = (int)n64;
    mps_graph *g = new (std::nothrow) mps_graph;
    if (!g) return MPS_ERR_UNSUPPORTED;
    try {
        // counting sort by row, then every row sorted and stripped of repeats
        std::vector<int64_t> start((size_t)n + 1, 0);
        for (int64_t e = 0; e < n_edges; ++e) ++start[(size_t)src[e] + 1];
        for (int i = 0; i < n; ++i) start[(size_t)i + 1] += start[(size_t)i];
        std::vector<int> cols((size_t)n_edges);
        {
            std::vector<int64_t> at(start.begin(), start.end() - 1);
            for (int64_t e = 0; e < n_edges; ++e) cols[(size_t)at[(size_t)src[e]]++] = (int)dst[e];
        }
        std::vector<int> kept((size_t)n, 0);
        parallel_for(n, 1 << 12, [&](int64_t lo, int64_t hi) {
            for (int64_t r = lo; r < hi; ++r) {
                int *b = cols.data() + start[(size_t)r], *e = cols.data() + start[(size_t)r + 1];
                std::sort(b, e);
                kept[(size_t)r] = (int)(std::unique(b, e) - b);
            }
        });
        g->row_ptr.resize((size_t)n + 1);
        g->row_ptr[0] = 0;
        for (int r = 0; r < n; ++r) g->row_ptr[(size_t)r + 1] = g->row_ptr[(size_t)r] + kept[(size_t)r];
        g->col_idx.resize((size_t)g->row_ptr[(size_t)n]);
        parallel_for(n, 1 << 12, [&](int64_t lo, int64_t hi) {
            for (int64_t r = lo; r < hi; ++r)
                std::copy(cols.data() + start[(size_t)r], cols.data() + start[(size_t)r] + kept[(size_t)r],
                          g->col_idx.data() + g->row_ptr[(size_t)r]);
        });
    } catch (const std::bad_alloc &) {
        delete g;
        return MPS_ERR_UNSUPPORTED;
    }
    finish_graph(g);
    *graph_out = g;
    return MPS_OK;
}

int mps_graph_from_csr_file(const char *path, mps_graph **graph_out)
{
    if (!path || !graph_out) return MPS_ERR_INVALID_ARG;
    *graph_out = nullptr;
    mps_graph *g = nullptr;
    try {
        std::vector<char> buf;
        if (!read_whole_file(path, buf)) return MPS_ERR_IO;
        int n = 0, nnz = 0;
        int rc = header_from_buf(buf, &n, &nnz);
        if (rc != MPS_OK) return rc;
        g = new mps_graph;
        g->row_ptr.resize((size_t)n + 1);
        g->col_idx.resize((size_t)nnz);
        rc = parse_csr(buf, n, nnz, g->row_ptr.data(), g->col_idx.data());
        if (rc != MPS_OK) {
            delete g;
            return rc;
        }
    } catch (const std::bad_alloc &) {
        delete g;
        return MPS_ERR_UNSUPPORTED;
    }
    finish_graph(g);
    *graph_out = g;
    return MPS_OK;
}

int mps_graph_dims(const mps_graph *g, int *n_rows_out, int *nnz_out, int *max_degree_out)
{
    if (!g) return MPS_ERR_INVALID_ARG;
    if (n_rows_out) *n_rows_out = (int)g->row_ptr.size() - 1;
    if (nnz_out) *nnz_out = (int)g->col_idx.size();
    if (max_degree_out) *max_degree_out = g->max_degree;
    return MPS_OK;
}

const int *mps_graph_row_ptr(const mps_graph *g) { return g ? g->row_ptr.data() : nullptr; }
const int *mps_graph_col_idx(const mps_graph *g) { return g ? g->col_idx.data() : nullptr; }
void mps_graph_free(mps_graph *g) { delete g; }

int mps_fill_uniform_f32(float *out, size_t n, uint64_t seed, float lo, float hi)
{
    if (!out && n) return MPS_ERR_INVALID_ARG;
    const uint64_t base = mix64(seed ^ 0xf1e2d3c4b5a69788ULL);
    const float span = hi - lo;
    parallel_for((int64_t)n, 1 << 18, [&](int64_t a, int64_t b) {
        for (int64_t i = a; i < b; ++i) {
            uint64_t r = mix64(base + (uint64_t)i * 0x9e3779b97f4a7c15ULL);
            float u = (float)(r >> 40) * (1.0f / 16777216.0f);
            out[i] = lo + span * u;
        }
    });
    return MPS_OK;
}

int mps_fill_uniform_f16(uint16_t *out, size_t n, uint64_t seed, float lo, float hi)
{
    if (!out && n) return MPS_ERR_INVALID_ARG;
    const uint64_t base = mix64(seed ^ 0xf1e2d3c4b5a69788ULL);
    const float span = hi - lo;
    parallel_for((int64_t)n, 1 << 18, [&](int64_t a, int64_t b) {
        for (int64_t i = a; i < b; ++i) {
            uint64_t r = mix64(base + (uint64_t)i * 0x9e3779b97f4a7c15ULL);
            float u = (float)(r >> 53) * (1.0f / 2048.0f);
            out[i] = float_to_half_bits(lo + span * u);
        }
    });
    return MPS_OK;
}

}  // extern "C"
