// npz_to_csr --graph <in.npz> --output <out.csr>
//
// Native counterpart of the reference's scripts/npz_to_csr.py (same two
// options, :8-11): reads the edge list of a GNNAdvisor .npz archive (arrays
// src_li and dst_li, :13-15), builds the CSR matrix the way
// coo_matrix(...).tocsr() does (:17-19: rows sorted, repeated edges merged) and
// writes the two-line comma-separated .csr text (:21-28).  No Python, numpy or
// scipy needed.  An .npz file is a zip archive of .npy members, stored
// (numpy.savez) or deflated (numpy.savez_compressed); integer arrays of 4 or 8
// bytes, little-endian, one dimension, are accepted.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include <zlib.h>

#include "mpspmm.h"

namespace {

[[noreturn]] void die(const std::string &msg)
{
    std::fprintf(stderr, "npz_to_csr: %s\n", msg.c_str());
    std::exit(1);
}

uint32_t rd16(const unsigned char *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }
uint32_t rd32(const unsigned char *p) { return rd16(p) | (rd16(p + 2) << 16); }
uint64_t rd64(const unsigned char *p) { return (uint64_t)rd32(p) | ((uint64_t)rd32(p + 4) << 32); }

struct Member {
    std::string name;
    int method = 0;
    uint64_t comp = 0, raw = 0, local = 0;
};

std::vector<unsigned char> read_file(const char *path)
{
    FILE *f = std::fopen(path, "rb");
    if (!f) die(std::string("cannot open ") + path);
    std::fseek(f, 0, SEEK_END);
    long sz = std::ftell(f);
    std::rewind(f);
    std::vector<unsigned char> buf(sz > 0 ? (size_t)sz : 0);
    if (sz > 0 && std::fread(buf.data(), 1, buf.size(), f) != buf.size()) die(std::string("cannot read ") + path);
    std::fclose(f);
    return buf;
}

// Central directory of the archive (sizes and offsets are taken from there:
// numpy writes local headers in zip64 form with the sizes in an extra field).
std::vector<Member> list_members(const std::vector<unsigned char> &z)
{
    if (z.size() < 22) die("not a zip archive");
    size_t eocd = z.size() - 22;
    for (;; --eocd) {
        if (rd32(&z[eocd]) == 0x06054b50u) break;
        if (eocd == 0 || z.size() - eocd > 22 + 65535) die("no end-of-central-directory record");
    }
    uint64_t count = rd16(&z[eocd + 10]), cd_off = rd32(&z[eocd + 16]);
    if (count == 0xffff || cd_off == 0xffffffffu) {  // zip64 end record
        if (eocd < 20 || rd32(&z[eocd - 20]) != 0x07064b50u) die("zip64 locator missing");
        uint64_t e64 = rd64(&z[eocd - 20 + 8]);
        if (e64 + 56 > z.size() || rd32(&z[e64]) != 0x06064b50u) die("zip64 end record missing");
        count = rd64(&z[e64 + 32]);
        cd_off = rd64(&z[e64 + 48]);
    }
    std::vector<Member> out;
    size_t p = (size_t)cd_off;
    for (uint64_t i = 0; i < count; ++i) {
        if (p + 46 > z.size() || rd32(&z[p]) != 0x02014b50u) die("damaged central directory");
        Member m;
        m.method = (int)rd16(&z[p + 10]);
        m.comp = rd32(&z[p + 20]);
        m.raw = rd32(&z[p + 24]);
        const size_t nlen = rd16(&z[p + 28]), xlen = rd16(&z[p + 30]), clen = rd16(&z[p + 32]);
        m.local = rd32(&z[p + 42]);
        if (p + 46 + nlen + xlen > z.size()) die("damaged central directory");
        m.name.assign(reinterpret_cast<const char *>(&z[p + 46]), nlen);
        // zip64 extra field: the values that did not fit, in the order raw, comp, local
        size_t x = p + 46 + nlen, xe = x + xlen;
        while (x + 4 <= xe) {
            const uint32_t id = rd16(&z[x]), len = rd16(&z[x + 2]);
            if (id == 1) {
                size_t q = x + 4;
                if (m.raw == 0xffffffffu && q + 8 <= xe) { m.raw = rd64(&z[q]); q += 8; }
                if (m.comp == 0xffffffffu && q + 8 <= xe) { m.comp = rd64(&z[q]); q += 8; }
                if (m.local == 0xffffffffu && q + 8 <= xe) { m.local = rd64(&z[q]); q += 8; }
            }
            x += 4 + len;
        }
        out.push_back(m);
        p += 46 + nlen + xlen + clen;
    }
    return out;
}

std::vector<unsigned char> extract(const std::vector<unsigned char> &z, const Member &m)
{
    if (m.local + 30 > z.size() || rd32(&z[m.local]) != 0x04034b50u) die("damaged local header of " + m.name);
    const size_t data = (size_t)m.local + 30 + rd16(&z[m.local + 26]) + rd16(&z[m.local + 28]);
    if (data + m.comp > z.size()) die("member " + m.name + " is cut short");
    std::vector<unsigned char> out((size_t)m.raw);
    if (m.method == 0) {
        if (m.comp != m.raw) die("stored member " + m.name + " has two sizes");
        std::memcpy(out.data(), &z[data], out.size());
    } else if (m.method == 8) {
        z_stream zs;
        std::memset(&zs, 0, sizeof zs);
        if (inflateInit2(&zs, -15) != Z_OK) die("zlib init failed");
        size_t in_done = 0, out_done = 0;
        int rc = Z_OK;
        while (rc != Z_STREAM_END) {  // 1 GiB at a time: zlib counts in 32 bits
            const size_t in_now = std::min<size_t>((size_t)m.comp - in_done, 1u << 30);
            const size_t out_now = std::min<size_t>(out.size() - out_done, 1u << 30);
            zs.next_in = const_cast<unsigned char *>(&z[data + in_done]);
            zs.avail_in = (uInt)in_now;
            zs.next_out = out.data() + out_done;
            zs.avail_out = (uInt)out_now;
            rc = inflate(&zs, Z_NO_FLUSH);
            if (rc != Z_OK && rc != Z_STREAM_END) die("cannot inflate " + m.name);
            in_done += in_now - zs.avail_in;
            out_done += out_now - zs.avail_out;
            if (rc == Z_OK && in_now - zs.avail_in == 0 && out_now - zs.avail_out == 0) die("cannot inflate " + m.name);
        }
        inflateEnd(&zs);
        if (out_done != out.size()) die("member " + m.name + " inflates to another size");
    } else {
        die("member " + m.name + ": compression method " + std::to_string(m.method) + " is not supported");
    }
    return out;
}

// .npy member -> int64 values (format 1.0 / 2.0 / 3.0 headers).
std::vector<int64_t> npy_integers(const std::vector<unsigned char> &b, const std::string &name)
{
    if (b.size() < 10 || std::memcmp(b.data(), "\x93NUMPY", 6) != 0) die(name + " is not an .npy array");
    const int major = b[6];
    size_t hlen, hoff;
    if (major == 1) { hlen = rd16(&b[8]); hoff = 10; }
    else if (major == 2 || major == 3) { if (b.size() < 12) die(name + ": short header"); hlen = rd32(&b[8]); hoff = 12; }
    else die(name + ": unknown .npy version");
    if (hoff + hlen > b.size()) die(name + ": short header");
    const std::string h(reinterpret_cast<const char *>(&b[hoff]), hlen);
    auto value_after = [&](const char *key) -> std::string {
        size_t k = h.find(key);
        if (k == std::string::npos) die(name + ": header has no " + key);
        k = h.find(':', k);
        size_t e = h.find_first_of(",}", k);
        if (h.find('(', k) < e) e = h.find(')', k) + 1;
        std::string v = h.substr(k + 1, e - k - 1);
        while (!v.empty() && (v.front() == ' ')) v.erase(v.begin());
        while (!v.empty() && (v.back() == ' ')) v.pop_back();
        return v;
    };
    std::string descr = value_after("'descr'");
    if (descr.size() >= 2 && (descr.front() == '\'' || descr.front() == '"')) descr = descr.substr(1, descr.size() - 2);
    if (value_after("'fortran_order'") != "False") die(name + ": Fortran order is not supported");
    const std::string shape = value_after("'shape'");
    int dims = 0;
    uint64_t count = 1;
    for (size_t i = 0; i < shape.size();) {
        if (shape[i] >= '0' && shape[i] <= '9') {
            uint64_t v = 0;
            while (i < shape.size() && shape[i] >= '0' && shape[i] <= '9') v = v * 10 + (uint64_t)(shape[i++] - '0');
            count *= v;
            ++dims;
        } else {
            ++i;
        }
    }
    if (dims != 1) die(name + ": expected a one-dimensional array, shape is " + shape);
    int width = 0;
    bool is_signed = true;
    if (descr == "<i8") width = 8;
    else if (descr == "<i4") width = 4;
    else if (descr == "<u8") { width = 8; is_signed = false; }
    else if (descr == "<u4") { width = 4; is_signed = false; }
    else die(name + ": element type " + descr + " is not supported (little-endian 4- or 8-byte integers are)");
    const unsigned char *d = &b[hoff + hlen];
    if (hoff + hlen + count * (uint64_t)width > b.size()) die(name + ": data is cut short");
    std::vector<int64_t> out((size_t)count);
    for (size_t i = 0; i < out.size(); ++i) {
        if (width == 8) out[i] = (int64_t)rd64(d + 8 * i);
        else out[i] = is_signed ? (int64_t)(int32_t)rd32(d + 4 * i) : (int64_t)rd32(d + 4 * i);
        if (!is_signed && out[i] < 0) die(name + ": value out of range");
    }
    return out;
}

}  // namespace

int main(int argc, char **argv)
{
    std::string in, out;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--graph" && i + 1 < argc) in = argv[++i];
        else if (a == "--output" && i + 1 < argc) out = argv[++i];
        else if (a.rfind("--graph=", 0) == 0) in = a.substr(8);
        else if (a.rfind("--output=", 0) == 0) out = a.substr(9);
        else die("usage: npz_to_csr --graph <in.npz> --output <out.csr>");
    }
    if (in.empty() || out.empty()) die("usage: npz_to_csr --graph <in.npz> --output <out.csr>");
    const std::vector<unsigned char> zip = read_file(in.c_str());
    std::vector<int64_t> src, dst;
    bool have_src = false, have_dst = false;
    for (const Member &m : list_members(zip)) {
        if (m.name == "src_li.npy") { src = npy_integers(extract(zip, m), m.name); have_src = true; }
        if (m.name == "dst_li.npy") { dst = npy_integers(extract(zip, m), m.name); have_dst = true; }
    }
    if (!have_src || !have_dst) die("the archive has no src_li / dst_li arrays");
    if (src.size() != dst.size()) die("src_li and dst_li differ in length");
    mps_graph *g = nullptr;
    int rc = mps_graph_from_edges(src.data(), dst.data(), (int64_t)src.size(), &g);
    if (rc != MPS_OK) die(std::string("mps_graph_from_edges: ") + mps_status_string(rc));
    int n = 0, nnz = 0, maxdeg = 0;
    mps_graph_dims(g, &n, &nnz, &maxdeg);
    rc = mps_csr_write(out.c_str(), n, mps_graph_row_ptr(g), mps_graph_col_idx(g));
    mps_graph_free(g);
    if (rc != MPS_OK) die(std::string("mps_csr_write: ") + mps_status_string(rc));
    std::printf("%s: %zu edges -> %d rows, %d non-zeros, max row degree %d -> %s\n", in.c_str(), src.size(), n, nnz, maxdeg,
                out.c_str());
    return 0;
}
