// .npy / .npz reader (zip central directory walk; stored and deflated members;
// zip64 extra fields as numpy writes them).
#include <zlib.h>

#include <cstdint>
#include <cstring>
#include <fstream>
#include <sstream>

#include "et/npy.hpp"

namespace et {
namespace npy {
namespace {

uint16_t rd16(const unsigned char *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
uint32_t rd32(const unsigned char *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
uint64_t rd64(const unsigned char *p) { return (uint64_t)rd32(p) | ((uint64_t)rd32(p + 4) << 32); }

std::vector<char> read_file(const std::string &path) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) throw Error(ET_ERR_IO, "cannot open " + path);
    const std::streamsize n = f.tellg();
    f.seekg(0);
    std::vector<char> buf((std::size_t)n);
    if (n > 0 && !f.read(buf.data(), n)) throw Error(ET_ERR_IO, "cannot read " + path);
    return buf;
}

[[noreturn]] void bad(const std::string &what, const std::string &why) {
    throw Error(ET_ERR_IO, what + ": " + why);
}

// value of key in the header dict text, e.g. find "'descr':" -> "'<f4'"
std::string dict_value(const std::string &hdr, const std::string &key, const std::string &what) {
    const std::size_t k = hdr.find("'" + key + "'");
    if (k == std::string::npos) bad(what, "npy header lacks '" + key + "'");
    std::size_t p = hdr.find(':', k);
    if (p == std::string::npos) bad(what, "malformed npy header");
    p++;
    while (p < hdr.size() && hdr[p] == ' ') p++;
    std::size_t e = p;
    if (hdr[p] == '(') {
        e = hdr.find(')', p);
        if (e == std::string::npos) bad(what, "malformed shape");
        return hdr.substr(p, e - p + 1);
    }
    while (e < hdr.size() && hdr[e] != ',' && hdr[e] != '}') e++;
    std::string v = hdr.substr(p, e - p);
    while (!v.empty() && v.back() == ' ') v.pop_back();
    return v;
}

std::vector<char> inflate_raw(const unsigned char *src, std::size_t clen, std::size_t ulen, const std::string &what) {
    std::vector<char> out(ulen);
    z_stream zs;
    std::memset(&zs, 0, sizeof zs);
    if (inflateInit2(&zs, -MAX_WBITS) != Z_OK) bad(what, "zlib init failed");
    zs.next_in = const_cast<unsigned char *>(src);
    zs.avail_in = (uInt)clen;
    zs.next_out = reinterpret_cast<unsigned char *>(out.data());
    zs.avail_out = (uInt)ulen;
    const int rc = inflate(&zs, Z_FINISH);
    inflateEnd(&zs);
    if (rc != Z_STREAM_END || zs.total_out != ulen) bad(what, "deflate stream is corrupt");
    return out;
}

}  // namespace

Array parse_npy(const char *buf, std::size_t len, const std::string &what) {
    const unsigned char *p = reinterpret_cast<const unsigned char *>(buf);
    if (len < 10 || std::memcmp(buf, "\x93NUMPY", 6) != 0) bad(what, "not an npy array");
    const int major = p[6];
    std::size_t hlen, hoff;
    if (major == 1) {
        hlen = rd16(p + 8);
        hoff = 10;
    } else if (major == 2 || major == 3) {
        if (len < 12) bad(what, "truncated npy header");
        hlen = rd32(p + 8);
        hoff = 12;
    } else {
        bad(what, "unsupported npy version");
    }
    if (hoff + hlen > len) bad(what, "truncated npy header");
    const std::string hdr(buf + hoff, hlen);
    Array a;
    std::string descr = dict_value(hdr, "descr", what);
    if (descr.size() < 4 || descr.front() != '\'') bad(what, "structured dtypes are not supported");
    a.descr = descr.substr(1, descr.size() - 2);
    if (a.descr[0] == '>') bad(what, "big-endian arrays are not supported");
    a.word_size = (std::size_t)std::stoul(a.descr.substr(2));
    a.fortran_order = dict_value(hdr, "fortran_order", what) == "True";
    std::string shape = dict_value(hdr, "shape", what);
    std::size_t i = 1;
    while (i < shape.size()) {
        while (i < shape.size() && (shape[i] == ' ' || shape[i] == ',')) i++;
        if (i >= shape.size() || shape[i] == ')') break;
        std::size_t e = i;
        while (e < shape.size() && shape[e] >= '0' && shape[e] <= '9') e++;
        if (e == i) bad(what, "malformed shape");
        a.shape.push_back((std::size_t)std::stoull(shape.substr(i, e - i)));
        i = e;
    }
    // the element count times the word size must not wrap: a shape whose product overflows would
    // pass the length test below
    const std::size_t avail = len - hoff - hlen;
    if (a.word_size == 0 || a.word_size > 16) bad(what, "unsupported element size");
    std::size_t count = 1;
    for (std::size_t d : a.shape) {
        if (d != 0 && count > avail / d) bad(what, "npy data shorter than its shape");
        count *= d;
    }
    if (count > avail / a.word_size) bad(what, "npy data shorter than its shape");
    const std::size_t nbytes = count * a.word_size;
    a.bytes.assign(buf + hoff + hlen, buf + hoff + hlen + nbytes);
    return a;
}

void npy_save(const std::string &path, const void *data, const std::string &descr, std::size_t word_size,
              const std::vector<std::size_t> &shape) {
    std::string dict = "{'descr': '" + descr + "', 'fortran_order': False, 'shape': (";
    std::size_t n = 1;
    for (std::size_t i = 0; i < shape.size(); i++) {
        dict += std::to_string(shape[i]) + (shape.size() == 1 || i + 1 < shape.size() ? "," : "");
        if (i + 1 < shape.size()) dict += " ";
        n *= shape[i];
    }
    dict += "), }";
    while ((10 + dict.size() + 1) % 64 != 0) dict += ' ';
    dict += '\n';
    std::ofstream f(path, std::ios::binary);
    if (!f) throw Error(ET_ERR_IO, "cannot create " + path);
    const unsigned char head[10] = {0x93, 'N', 'U', 'M', 'P', 'Y', 1, 0, (unsigned char)(dict.size() & 0xff),
                                    (unsigned char)(dict.size() >> 8)};
    f.write(reinterpret_cast<const char *>(head), 10);
    f.write(dict.data(), (std::streamsize)dict.size());
    f.write(static_cast<const char *>(data), (std::streamsize)(n * word_size));
    if (!f) throw Error(ET_ERR_IO, "cannot write " + path);
}

Array npy_load(const std::string &path) {
    const std::vector<char> buf = read_file(path);
    return parse_npy(buf.data(), buf.size(), path);
}

npz_t npz_load(const std::string &path) {
    const std::vector<char> file = read_file(path);
    const unsigned char *p = reinterpret_cast<const unsigned char *>(file.data());
    const std::size_t n = file.size();
    if (n < 22) bad(path, "not a zip archive");
    // end-of-central-directory record: scan back over a possible comment
    std::size_t eocd = std::string::npos;
    for (std::size_t i = n - 22 + 1; i-- > 0;) {
        if (rd32(p + i) == 0x06054b50u) {
            eocd = i;
            break;
        }
        if (n - i > 22 + 65535) break;
    }
    if (eocd == std::string::npos) bad(path, "zip end record not found");
    uint64_t entries = rd16(p + eocd + 10);
    uint64_t cd_off = rd32(p + eocd + 16);
    if (entries == 0xFFFF || cd_off == 0xFFFFFFFFu) {
        // zip64: locator sits right before the end record
        if (eocd < 20 || rd32(p + eocd - 20) != 0x07064b50u) bad(path, "zip64 locator missing");
        const uint64_t e64 = rd64(p + eocd - 20 + 8);
        if (e64 > n || n - e64 < 56 || rd32(p + e64) != 0x06064b50u) bad(path, "zip64 end record missing");
        entries = rd64(p + e64 + 32);
        cd_off = rd64(p + e64 + 48);
    }
    npz_t out;
    if (cd_off > n) bad(path, "zip central directory lies outside the file");
    std::size_t pos = (std::size_t)cd_off;
    for (uint64_t e = 0; e < entries; e++) {
        if (pos > n || n - pos < 46 || rd32(p + pos) != 0x02014b50u) bad(path, "zip central directory is corrupt");
        const uint16_t method = rd16(p + pos + 10);
        uint64_t csize = rd32(p + pos + 20), usize = rd32(p + pos + 24);
        const uint16_t nlen = rd16(p + pos + 28), xlen = rd16(p + pos + 30), clen = rd16(p + pos + 32);
        uint64_t lho = rd32(p + pos + 42);
        // name, extra field and comment of this entry must lie inside the file
        if (n - pos - 46 < (std::size_t)nlen + xlen + clen) bad(path, "zip central directory is corrupt");
        std::string name(file.data() + pos + 46, nlen);
        // zip64 extra field (id 1): the 64-bit values appear for each 32-bit field that is saturated
        std::size_t x = pos + 46 + nlen;
        const std::size_t xend = x + xlen;
        while (x + 4 <= xend) {
            const uint16_t id = rd16(p + x), sz = rd16(p + x + 2);
            if (x + 4 + (std::size_t)sz > xend) bad(path, "zip extra field is corrupt");
            if (id == 0x0001) {
                std::size_t q = x + 4;
                const std::size_t qend = x + 4 + sz;
                auto take64 = [&](uint64_t &v) {
                    if (q + 8 > qend) bad(path, "zip64 extra field is too short");
                    v = rd64(p + q);
                    q += 8;
                };
                if (usize == 0xFFFFFFFFu) take64(usize);
                if (csize == 0xFFFFFFFFu) take64(csize);
                if (lho == 0xFFFFFFFFu) take64(lho);
            }
            x += 4 + (std::size_t)sz;
        }
        pos = xend + clen;
        if (lho > n || n - lho < 30 || rd32(p + lho) != 0x04034b50u) bad(path, "zip local header is corrupt");
        const std::size_t data = (std::size_t)lho + 30 + rd16(p + lho + 26) + rd16(p + lho + 28);
        if (data > n || csize > n - data) bad(path, "zip member runs past the end of the file");
        if (usize > ((uint64_t)1 << 40)) bad(path, "zip member claims an implausible size");
        std::vector<char> raw;
        if (method == 0) {
            raw.assign(file.data() + data, file.data() + data + csize);
        } else if (method == 8) {
            raw = inflate_raw(p + data, (std::size_t)csize, (std::size_t)usize, path + ":" + name);
        } else {
            bad(path, "zip member " + name + " uses an unsupported compression method");
        }
        if (name.size() > 4 && name.compare(name.size() - 4, 4, ".npy") == 0) name.resize(name.size() - 4);
        out.emplace(name, parse_npy(raw.data(), raw.size(), path + ":" + name));
    }
    return out;
}

}  // namespace npy
}  // namespace et
