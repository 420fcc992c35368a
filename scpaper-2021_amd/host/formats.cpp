// Host construction of the sparse weight structures and their C-ABI exports.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <numeric>

#include "et/format_gen.h"
#include "et/status.h"

namespace et {
namespace fmt {

static inline uint64_t splitmix64_at(uint64_t seed, uint64_t index_from_one) {
    uint64_t z = seed + index_from_one * 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

std::vector<int64_t> permutation(int64_t n, uint64_t seed) {
    std::vector<uint64_t> key((size_t)n);
    for (int64_t i = 0; i < n; i++) key[(size_t)i] = splitmix64_at(seed, (uint64_t)i + 1);
    std::vector<int64_t> ids((size_t)n);
    std::iota(ids.begin(), ids.end(), (int64_t)0);
    std::stable_sort(ids.begin(), ids.end(),
                     [&](int64_t a, int64_t b) { return key[(size_t)a] < key[(size_t)b]; });
    return ids;
}

int kept_count(int64_t total, float sparsity) {
    return (int)((double)total * (1.0 - (double)sparsity));
}

// Groups permuted ids (x = id % stride, y = id / stride) by y, keeping the
// permuted order inside each group: the reference's copy_if-per-row.
static void group_by_row(const std::vector<int64_t> &kept, int64_t stride, int nrows,
                         std::vector<int> &ptr, std::vector<int> &xs) {
    ptr.assign((size_t)nrows + 1, 0);
    for (int64_t id : kept) ptr[(size_t)(id / stride) + 1]++;
    for (int r = 0; r < nrows; r++) ptr[(size_t)r + 1] += ptr[(size_t)r];
    xs.assign(kept.size(), 0);
    std::vector<int> cursor(ptr.begin(), ptr.end() - 1);
    for (int64_t id : kept) xs[(size_t)cursor[(size_t)(id / stride)]++] = (int)(id % stride);
}

TilePattern gen_tile_pattern(int nrow, int ncol, float sparsity, uint64_t seed) {
    const int br = nrow / kTile, bc = ncol / kTile;
    const int64_t total = (int64_t)br * bc;
    const int ntile = kept_count(total, sparsity);
    auto perm = permutation(total, seed);
    perm.resize((size_t)std::max<int64_t>(0, std::min<int64_t>(ntile, total)));
    TilePattern p;
    group_by_row(perm, bc, br, p.row_ptr, p.row_offset);
    return p;
}

TilePattern dense_tile_pattern(int nrow, int ncol) {
    const int br = nrow / kTile, bc = ncol / kTile;
    TilePattern p;
    p.row_ptr.resize((size_t)br + 1);
    for (int r = 0; r <= br; r++) p.row_ptr[(size_t)r] = r * bc;
    p.row_offset.resize((size_t)br * bc);
    for (int r = 0; r < br; r++)
        for (int c = 0; c < bc; c++) p.row_offset[(size_t)r * bc + c] = c;
    return p;
}

Bsr16 dense_to_bsr16(const float *W, int nrow, int ncol) {
    const int br = nrow / kTile, bc = ncol / kTile;
    Bsr16 m;
    m.row_ptr.push_back(0);
    for (int i = 0; i < br; i++) {
        for (int j = 0; j < bc; j++) {
            bool any = false;
            for (int r = 0; r < kTile && !any; r++)
                for (int c = 0; c < kTile; c++)
                    if (W[(size_t)(i * kTile + r) * ncol + j * kTile + c] != 0.0f) {
                        any = true;
                        break;
                    }
            if (!any) continue;
            m.column.push_back(j);
            for (int r = 0; r < kTile; r++)
                for (int c = 0; c < kTile; c++)
                    m.data.push_back(W[(size_t)(i * kTile + r) * ncol + j * kTile + c]);
        }
        m.row_ptr.push_back((int)m.column.size());
    }
    return m;
}

std::vector<float> bsr16_to_dense(const int *row_ptr, const int *column, const float *data,
                                  int nrow, int ncol) {
    std::vector<float> W((size_t)nrow * ncol, 0.0f);
    for (int i = 0; i < nrow / kTile; i++)
        for (int t = row_ptr[i]; t < row_ptr[i + 1]; t++)
            for (int r = 0; r < kTile; r++)
                for (int c = 0; c < kTile; c++)
                    W[(size_t)(i * kTile + r) * ncol + column[t] * kTile + c] =
                        data[(size_t)t * 256 + r * kTile + c];
    return W;
}

void validate_bsr16(const std::vector<int> &row_ptr, const std::vector<int> &column,
                    std::size_t ntile, int blk_col_num) {
    require(!row_ptr.empty() && row_ptr.front() == 0, "tile_mat: row_ptr must start at 0");
    for (size_t i = 1; i < row_ptr.size(); i++)
        require(row_ptr[i] >= row_ptr[i - 1], "tile_mat: row_ptr must be non-decreasing");
    require((size_t)row_ptr.back() == ntile && column.size() == ntile,
            "tile_mat: row_ptr.back(), the column count and the tile count must agree");
    for (size_t t = 0; t < column.size(); t++) {
        const int c = column[t];
        if (c < 0 || c >= blk_col_num)
            throw Error(ET_ERR_INVALID_ARG, "tile_mat: column-tile index out of range (tile " + std::to_string(t) +
                                                " of " + std::to_string(ntile) + " has column " + std::to_string(c) +
                                                ", the matrix has " + std::to_string(blk_col_num) + " column tiles)");
    }
}

void validate_csr(const std::vector<int> &indptr, const std::vector<int> &indices, std::size_t ndata, int nrow,
                  int ncol) {
    require(nrow >= 0 && ncol >= 0 && indptr.size() == (size_t)nrow + 1, "csr_mat: indptr must hold nrow + 1 entries");
    require(indptr.front() == 0, "csr_mat: indptr must start at 0");
    for (size_t i = 1; i < indptr.size(); i++)
        require(indptr[i] >= indptr[i - 1], "csr_mat: indptr must be non-decreasing");
    require((size_t)indptr.back() == indices.size() && ndata == indices.size(),
            "csr_mat: indptr.back(), the index count and the value count must agree");
    for (int c : indices) require(c >= 0 && c < ncol, "csr_mat: column index out of range");
}

std::vector<int> gen_row_ids(int nrow, float sparsity, uint64_t seed) {
    int nn = kept_count(nrow, sparsity);
    nn = ((nn / 16) + ((nn % 16) != 0)) * 16;
    nn = std::max(0, std::min(nn, nrow));
    auto perm = permutation(nrow, seed);
    std::vector<int> ids(perm.begin(), perm.begin() + nn);
    std::sort(ids.begin(), ids.end());
    return ids;
}

std::vector<int> gen_col_ids(int ncol, float sparsity, uint64_t seed) {
    int nn = kept_count(ncol, sparsity);
    nn = 16 * (nn / 16);
    nn = std::max(0, std::min(nn, ncol));
    auto perm = permutation(ncol, seed);
    return std::vector<int>(perm.begin(), perm.begin() + nn);
}

std::vector<int> head_ptr(const std::vector<int> &col_id, int nnz_col, int nhead, int full_dim) {
    require(nhead > 0 && full_dim % nhead == 0, "head_ptr: full_dim must be a multiple of nhead");
    require(nnz_col >= 0 && (size_t)nnz_col <= col_id.size(), "head_ptr: nnz_col exceeds the id list");
    const int hd = full_dim / nhead;
    std::vector<int> out{0};
    for (int h = 0; h < nhead; h++) {
        const int hi = (h + 1) * hd;
        int i = out.back();
        while (i < nnz_col && col_id[(size_t)i] < hi) i++;
        out.push_back(i);
    }
    require(out.back() == nnz_col, "head_ptr: column ids must be ascending and below full_dim");
    return out;
}

static int pad16(int n) { return ((n + 15) / 16) * 16; }

Vec1x16 dense_to_1x16(const float *W, int nrow, int ncol) {
    const int npart = ncol / kTile;
    Vec1x16 m;
    int count = 0;
    for (int r = 0; r < nrow / kTile; r++) {
        for (int p = 0; p < npart; p++) {
            m.tile_idx.push_back(count);
            for (int i = 0; i < kTile; i++) {
                const float *vec = W + (size_t)(r * kTile + i) * ncol + p * kTile;
                bool any = false;
                for (int c = 0; c < kTile; c++) any = any || vec[c] != 0.0f;
                if (!any) continue;
                m.row_idx.push_back(r * kTile + i);
                m.data.insert(m.data.end(), vec, vec + kTile);
                count++;
            }
        }
        m.tile_idx.push_back(count);
    }
    m.data.resize((size_t)pad16(count) * kTile, 0.0f);
    return m;
}

Vec1x16 gen_1x16_pattern(int nrow, int ncol, float sparsity, uint64_t seed) {
    const int npart = ncol / kTile;
    const int64_t total = (int64_t)npart * nrow;
    const int ntile = kept_count(total, sparsity);
    auto perm = permutation(total, seed);
    perm.resize((size_t)std::max<int64_t>(0, std::min<int64_t>(ntile, total)));
    // cell = (row-set, part); keep the permuted order inside a cell
    const int nsets = nrow / kTile;
    std::vector<std::vector<int>> cells((size_t)nsets * npart);
    for (int64_t id : perm) {
        const int x = (int)(id % npart), y = (int)(id / npart);
        if (y / kTile < nsets) cells[(size_t)(y / kTile) * npart + x].push_back(y);
    }
    Vec1x16 m;
    int count = 0;
    for (int r = 0; r < nsets; r++) {
        for (int p = 0; p < npart; p++) {
            m.tile_idx.push_back(count);
            const auto &cell = cells[(size_t)r * npart + p];
            m.row_idx.insert(m.row_idx.end(), cell.begin(), cell.end());
            count += (int)cell.size();
        }
        m.tile_idx.push_back(count);
    }
    return m;
}

std::vector<float> vec1x16_to_dense(const Vec1x16 &m, int nrow, int ncol) {
    const int npart = ncol / kTile;
    std::vector<float> W((size_t)nrow * ncol, 0.0f);
    for (int r = 0; r < nrow / kTile; r++) {
        const int base = r * (npart + 1);
        for (int p = 0; p < npart; p++)
            for (int idx = m.tile_idx[(size_t)base + p]; idx < m.tile_idx[(size_t)base + p + 1]; idx++)
                for (int c = 0; c < kTile; c++)
                    W[(size_t)(r * kTile + m.row_idx[(size_t)idx] % kTile) * ncol + p * kTile + c] =
                        m.data[(size_t)idx * kTile + c];
    }
    return W;
}

Csr dense_to_csr(const float *W, int nrow, int ncol) {
    Csr m;
    m.nrow = nrow;
    m.ncol = ncol;
    m.indptr.push_back(0);
    for (int r = 0; r < nrow; r++) {
        for (int c = 0; c < ncol; c++) {
            const float v = W[(size_t)r * ncol + c];
            if (v != 0.0f) {
                m.indices.push_back(c);
                m.data.push_back(v);
            }
        }
        m.indptr.push_back((int)m.indices.size());
    }
    m.nnz = (int)m.indices.size();
    return m;
}

Csr gen_csr_pattern(int nrow, int ncol, float sparsity, uint64_t seed) {
    const int64_t total = (int64_t)nrow * ncol;
    const int nnz = kept_count(total, sparsity);
    auto perm = permutation(total, seed);
    perm.resize((size_t)std::max<int64_t>(0, std::min<int64_t>(nnz, total)));
    Csr m;
    m.nrow = nrow;
    m.ncol = ncol;
    m.nnz = (int)perm.size();
    group_by_row(perm, ncol, nrow, m.indptr, m.indices);
    m.data.assign(perm.size(), 1.0f);
    return m;
}

Csr read_csr(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw Error(ET_ERR_IO, "cannot open " + path);
    uint32_t head[3];
    f.read(reinterpret_cast<char *>(head), sizeof head);
    if (!f) throw Error(ET_ERR_IO, path + ": truncated header");
    Csr m;
    m.nrow = (int)head[0];
    m.ncol = (int)head[1];
    m.nnz = (int)head[2];
    // the header must describe the file before anything is sized from it
    f.seekg(0, std::ios::end);
    const uint64_t file_bytes = (uint64_t)f.tellg();
    f.seekg(12, std::ios::beg);
    if (m.nrow < 0 || m.ncol < 0 || m.nnz < 0 ||
        file_bytes != 12 + 4 * ((uint64_t)head[0] + 1) + 8 * (uint64_t)head[2])
        throw Error(ET_ERR_IO, path + ": header does not match the file size");
    m.indptr.resize((size_t)m.nrow + 1);
    m.indices.resize((size_t)m.nnz);
    m.data.resize((size_t)m.nnz);
    f.read(reinterpret_cast<char *>(m.indptr.data()), (std::streamsize)(m.indptr.size() * 4));
    f.read(reinterpret_cast<char *>(m.indices.data()), (std::streamsize)(m.indices.size() * 4));
    f.read(reinterpret_cast<char *>(m.data.data()), (std::streamsize)(m.data.size() * 4));
    if (!f) throw Error(ET_ERR_IO, path + ": truncated body");
    validate_csr(m.indptr, m.indices, m.data.size(), m.nrow, m.ncol);
    return m;
}

void write_csr(const std::string &path, const Csr &m) {
    std::ofstream f(path, std::ios::binary);
    if (!f) throw Error(ET_ERR_IO, "cannot create " + path);
    const uint32_t head[3] = {(uint32_t)m.nrow, (uint32_t)m.ncol, (uint32_t)m.nnz};
    f.write(reinterpret_cast<const char *>(head), sizeof head);
    f.write(reinterpret_cast<const char *>(m.indptr.data()), (std::streamsize)(m.indptr.size() * 4));
    f.write(reinterpret_cast<const char *>(m.indices.data()), (std::streamsize)(m.indices.size() * 4));
    f.write(reinterpret_cast<const char *>(m.data.data()), (std::streamsize)(m.data.size() * 4));
}

}  // namespace fmt
}  // namespace et

// --------------------------------------------------------------------------
// C ABI
// --------------------------------------------------------------------------
using namespace et;

namespace {
template <typename Fn> int guarded(Fn fn) {
    try {
        return fn();
    } catch (const Error &e) {
        et_set_last_error(e.what());
        return e.status();
    } catch (const std::exception &e) {
        et_set_last_error(e.what());
        return ET_ERR_INVALID_ARG;
    }
}
template <typename T> void copy_out(const std::vector<T> &v, T *dst) {
    if (dst && !v.empty()) std::memcpy(dst, v.data(), v.size() * sizeof(T));
}
bool dims16(int nrow, int ncol) { return nrow > 0 && ncol > 0 && nrow % 16 == 0 && ncol % 16 == 0; }
}  // namespace

extern "C" {

int et_fmt_permutation(int64_t n, uint64_t seed, int64_t *out) {
    return guarded([&]() -> int {
        require(n >= 0 && (out || n == 0), "et_fmt_permutation: bad arguments");
        copy_out(fmt::permutation(n, seed), out);
        return ET_OK;
    });
}

int et_fmt_kept_count(int64_t total, float sparsity) { return fmt::kept_count(total, sparsity); }

int et_fmt_tile_pattern(int nrow, int ncol, float sparsity, uint64_t seed, int32_t *row_ptr,
                        int32_t *row_offset, int *ntile) {
    return guarded([&]() -> int {
        require(dims16(nrow, ncol), "et_fmt_tile_pattern: dimensions must be positive multiples of 16");
        require(row_ptr && row_offset && ntile, "et_fmt_tile_pattern: NULL output");
        auto p = fmt::gen_tile_pattern(nrow, ncol, sparsity, seed);
        copy_out(p.row_ptr, row_ptr);
        copy_out(p.row_offset, row_offset);
        *ntile = (int)p.row_offset.size();
        return ET_OK;
    });
}

int et_fmt_dense_to_bsr16(const float *W, int nrow, int ncol, int32_t *row_ptr, int32_t *column,
                          float *data, int *ntile) {
    return guarded([&]() -> int {
        require(dims16(nrow, ncol), "et_fmt_dense_to_bsr16: dimensions must be positive multiples of 16");
        require(W && row_ptr && ntile, "et_fmt_dense_to_bsr16: NULL argument");
        auto m = fmt::dense_to_bsr16(W, nrow, ncol);
        copy_out(m.row_ptr, row_ptr);
        copy_out(m.column, column);  // column/data may be NULL to query the count
        copy_out(m.data, data);
        *ntile = (int)m.column.size();
        return ET_OK;
    });
}

int et_fmt_row_ids(int nrow, float sparsity, uint64_t seed, int32_t *ids, int *count) {
    return guarded([&]() -> int {
        require(nrow > 0 && count, "et_fmt_row_ids: bad arguments");
        auto v = fmt::gen_row_ids(nrow, sparsity, seed);
        copy_out(v, ids);
        *count = (int)v.size();
        return ET_OK;
    });
}

int et_fmt_col_ids(int ncol, float sparsity, uint64_t seed, int32_t *ids, int *count) {
    return guarded([&]() -> int {
        require(ncol > 0 && count, "et_fmt_col_ids: bad arguments");
        auto v = fmt::gen_col_ids(ncol, sparsity, seed);
        copy_out(v, ids);
        *count = (int)v.size();
        return ET_OK;
    });
}

int et_fmt_head_ptr(const int32_t *col_id, int nnz_col, int nhead, int full_dim, int32_t *out) {
    return guarded([&]() -> int {
        require(col_id && out && nnz_col >= 0, "et_fmt_head_ptr: bad arguments");
        std::vector<int> ids(col_id, col_id + nnz_col);
        copy_out(fmt::head_ptr(ids, nnz_col, nhead, full_dim), out);
        return ET_OK;
    });
}

int et_fmt_dense_to_1x16(const float *W, int nrow, int ncol, int32_t *tile_idx, int32_t *row_idx,
                         float *data, int *ntile) {
    return guarded([&]() -> int {
        require(dims16(nrow, ncol), "et_fmt_dense_to_1x16: dimensions must be positive multiples of 16");
        require(W && tile_idx && ntile, "et_fmt_dense_to_1x16: NULL argument");
        auto m = fmt::dense_to_1x16(W, nrow, ncol);
        copy_out(m.tile_idx, tile_idx);
        copy_out(m.row_idx, row_idx);
        copy_out(m.data, data);
        *ntile = (int)m.row_idx.size();
        return ET_OK;
    });
}

int et_fmt_1x16_pattern(int nrow, int ncol, float sparsity, uint64_t seed, int32_t *tile_idx,
                        int32_t *row_idx, int *ntile) {
    return guarded([&]() -> int {
        require(dims16(nrow, ncol), "et_fmt_1x16_pattern: dimensions must be positive multiples of 16");
        require(tile_idx && ntile, "et_fmt_1x16_pattern: NULL argument");
        auto m = fmt::gen_1x16_pattern(nrow, ncol, sparsity, seed);
        copy_out(m.tile_idx, tile_idx);
        copy_out(m.row_idx, row_idx);
        *ntile = (int)m.row_idx.size();
        return ET_OK;
    });
}

int et_fmt_dense_to_csr(const float *W, int nrow, int ncol, int32_t *indptr, int32_t *indices,
                        float *data, int *nnz) {
    return guarded([&]() -> int {
        require(W && indptr && nnz && nrow > 0 && ncol > 0, "et_fmt_dense_to_csr: bad arguments");
        auto m = fmt::dense_to_csr(W, nrow, ncol);
        copy_out(m.indptr, indptr);
        copy_out(m.indices, indices);
        copy_out(m.data, data);
        *nnz = m.nnz;
        return ET_OK;
    });
}

int et_fmt_csr_pattern(int nrow, int ncol, float sparsity, uint64_t seed, int32_t *indptr,
                       int32_t *indices, int *nnz) {
    return guarded([&]() -> int {
        require(indptr && nnz && nrow > 0 && ncol > 0, "et_fmt_csr_pattern: bad arguments");
        auto m = fmt::gen_csr_pattern(nrow, ncol, sparsity, seed);
        copy_out(m.indptr, indptr);
        copy_out(m.indices, indices);
        *nnz = m.nnz;
        return ET_OK;
    });
}

int et_fmt_csr_read(const char *path, int *nrow, int *ncol, int *nnz, int32_t *indptr,
                    int32_t *indices, float *data) {
    return guarded([&]() -> int {
        require(path && nrow && ncol && nnz, "et_fmt_csr_read: NULL argument");
        auto m = fmt::read_csr(path);
        *nrow = m.nrow;
        *ncol = m.ncol;
        *nnz = m.nnz;
        copy_out(m.indptr, indptr);  // NULL on the sizing call
        copy_out(m.indices, indices);
        copy_out(m.data, data);
        return ET_OK;
    });
}

}  // extern "C"
