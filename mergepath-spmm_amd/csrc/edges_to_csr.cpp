// edges_to_csr --edges <in.txt> --output <out.csr> [--undirected]
//
// Text edge list -> the two-line comma-separated .csr text the drivers read.
// What scripts/fetch_dataset.py:10-21 does for a PyTorch Geometric dataset
// (edge_index -> to_scipy_sparse_matrix -> tocsr -> the write loop), for edge
// lists that are already on disk, e.g. the SNAP and SuiteSparse graphs of the
// reference's README (amazon0505, com-amazon, soc-BlogCatalog ...): one edge
// "src dst" per line, separated by blanks, tabs or a comma; lines that start
// with '#' or '%' are comments; anything after the second number of a line
// (a weight, a time stamp) is ignored.  Rows are sorted, repeated edges merged
// (scipy's coo -> csr); the matrix is square with max id + 1 rows.
// --undirected also stores every edge the other way round.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "mpspmm.h"

namespace {

[[noreturn]] void die(const std::string &msg)
{
    std::fprintf(stderr, "edges_to_csr: %s\n", msg.c_str());
    std::exit(1);
}

// Next non-negative integer at p (blanks, tabs and one comma skipped first); false at the end of the line.
bool next_id(const char *&p, const char *end, int64_t &out)
{
    while (p < end && (*p == ' ' || *p == '\t' || *p == ',' || *p == '\r')) ++p;
    if (p >= end || *p == '\n') return false;
    if (*p < '0' || *p > '9') die("malformed line: expected a non-negative integer");
    int64_t v = 0;
    while (p < end && *p >= '0' && *p <= '9') {
        v = v * 10 + (*p - '0');
        if (v > 0x7fffffffLL) die("node id beyond 32 bits");
        ++p;
    }
    out = v;
    return true;
}

}  // namespace

int main(int argc, char **argv)
{
    const char *in = nullptr, *out = nullptr;
    bool undirected = false;
    for (int i = 1; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--edges") && i + 1 < argc) in = argv[++i];
        else if (!std::strcmp(argv[i], "--output") && i + 1 < argc) out = argv[++i];
        else if (!std::strcmp(argv[i], "--undirected")) undirected = true;
        else die(std::string("unknown argument ") + argv[i]);
    }
    if (!in || !out) {
        std::fprintf(stderr, "Usage: edges_to_csr --edges <in.txt> --output <out.csr> [--undirected]\n");
        return 1;
    }
    FILE *f = std::fopen(in, "rb");
    if (!f) die(std::string("cannot open ") + in);
    std::fseek(f, 0, SEEK_END);
    const long sz = std::ftell(f);
    std::rewind(f);
    std::vector<char> buf(sz > 0 ? (size_t)sz : 0);
    if (sz > 0 && std::fread(buf.data(), 1, buf.size(), f) != buf.size()) die(std::string("cannot read ") + in);
    std::fclose(f);

    std::vector<int64_t> src, dst;
    const char *p = buf.data(), *end = buf.data() + buf.size();
    while (p < end) {
        const char *nl = static_cast<const char *>(std::memchr(p, '\n', (size_t)(end - p)));
        const char *line_end = nl ? nl : end;
        const char *q = p;
        while (q < line_end && (*q == ' ' || *q == '\t')) ++q;
        if (q < line_end && *q != '#' && *q != '%' && *q != '\r') {
            int64_t a = 0, b = 0;
            if (!next_id(q, line_end, a) || !next_id(q, line_end, b)) die("malformed line: two node ids expected");
            src.push_back(a);
            dst.push_back(b);
            if (undirected && a != b) {
                src.push_back(b);
                dst.push_back(a);
            }
        }
        p = nl ? nl + 1 : end;
    }
    mps_graph *g = nullptr;
    int rc = mps_graph_from_edges(src.data(), dst.data(), (int64_t)src.size(), &g);
    if (rc != MPS_OK) die(std::string("mps_graph_from_edges: ") + mps_status_string(rc));
    int n = 0, nnz = 0, max_degree = 0;
    mps_graph_dims(g, &n, &nnz, &max_degree);
    rc = mps_csr_write(out, n, mps_graph_row_ptr(g), mps_graph_col_idx(g));
    if (rc != MPS_OK) die(std::string("cannot write ") + out);
    std::printf("%d rows, %d nonzeros (from %zu edges read), max row degree %d\n", n, nnz, src.size(), max_degree);
    mps_graph_free(g);
    return 0;
}
