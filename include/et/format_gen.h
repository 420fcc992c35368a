// Host-side construction of the sparse weight structures (integer work, no GPU).
// Implemented in scpaper-2021_amd/host/formats.cpp; the same functions are
// exported through the C ABI (et_fmt_*) so that other languages and the tests
// can reach them.
//
// Random structure: the reference permutes ids with std::random_shuffle over
// rand() (mat_type/tile_mat/tile_mat.cu:16 and the other generators), which is
// not reproducible.  Here the permutation is seeded: id i gets the SplitMix64
// key number i+1 of the stream started at `seed`, and ids are taken in ascending
// key order (ties by id).  Every other step — counts, truncation, grouping,
// ordering — follows the reference generator cited at each function.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace et {
namespace fmt {

constexpr int kTile = 16;
constexpr uint64_t kDefaultSeed = 0x5eed5eedULL;

std::vector<int64_t> permutation(int64_t n, uint64_t seed);

// int(total * (1.0 - sparsity)) with the float promoted to double
// (mat_type/tile_mat/tile_mat.cu:12).
int kept_count(int64_t total, float sparsity);

struct TilePattern {
    std::vector<int> row_ptr;     // [nrow/16 + 1]
    std::vector<int> row_offset;  // [ntile] column-tile index of each tile
};
// tile_mat::gen_sparse_mat structure (mat_type/tile_mat/tile_mat.cu:7-40).
TilePattern gen_tile_pattern(int nrow, int ncol, float sparsity, uint64_t seed);
// tile_mat::gen_dense_mat structure (mat_type/tile_mat/tile_mat.cu:42-64).
TilePattern dense_tile_pattern(int nrow, int ncol);

struct Bsr16 {
    std::vector<int> row_ptr, column;
    std::vector<float> data;  // [ntile][256], tile row-major, rows = output features
};
// Exporter semantics (example/npy2pt.py:75-109).
Bsr16 dense_to_bsr16(const float *W, int nrow, int ncol);
std::vector<float> bsr16_to_dense(const int *row_ptr, const int *column, const float *data,
                                  int nrow, int ncol);
// Throws et::Error unless row_ptr is monotone from 0 to ntile and every column
// index lies in [0, blk_col_num).
void validate_bsr16(const std::vector<int> &row_ptr, const std::vector<int> &column,
                    std::size_t ntile, int blk_col_num);

// CSR consistency: indptr[nrow+1] starting at 0 and non-decreasing, indptr.back() == index count
// == value count, every column inside [0, ncol).  Throws et::Error otherwise.
void validate_csr(const std::vector<int> &indptr, const std::vector<int> &indices, std::size_t ndata, int nrow,
                  int ncol);

// row_mat::gen_sparse_mat ids (mat_type/row_mat/row_mat.cu:14-25): ascending.
std::vector<int> gen_row_ids(int nrow, float sparsity, uint64_t seed);
// col_mat::gen_sparse_mat ids (mat_type/col_mat/col_mat.cu:22-32): permuted order.
std::vector<int> gen_col_ids(int ncol, float sparsity, uint64_t seed);
// col_mat::set_metadata (mat_type/col_mat/col_mat.cu:34-58).
std::vector<int> head_ptr(const std::vector<int> &col_id, int nnz_col, int nhead, int full_dim);

struct Vec1x16 {
    std::vector<int> tile_idx;  // [(nrow/16) * (ncol/16 + 1)] global offsets
    std::vector<int> row_idx;   // [ntile] absolute row of each 1x16 vector
    std::vector<float> data;    // [pad16(ntile)][16]
};
// Layout read by the reference kernel (Linear/SPMM1x16.cu:52-74).
Vec1x16 dense_to_1x16(const float *W, int nrow, int ncol);
Vec1x16 gen_1x16_pattern(int nrow, int ncol, float sparsity, uint64_t seed);  // data left empty
std::vector<float> vec1x16_to_dense(const Vec1x16 &m, int nrow, int ncol);

struct Csr {
    std::vector<int> indptr, indices;
    std::vector<float> data;
    int nrow = 0, ncol = 0, nnz = 0;
};
Csr dense_to_csr(const float *W, int nrow, int ncol);
// csr_mat::gen_sparse_mat structure (mat_type/csr_mat/csr_mat.cpp:25-67), column = id % ncol.
Csr gen_csr_pattern(int nrow, int ncol, float sparsity, uint64_t seed);
// .csr file (mat_type/csr_mat/csr_mat.h:19-35).
Csr read_csr(const std::string &path);
void write_csr(const std::string &path, const Csr &m);

}  // namespace fmt
}  // namespace et
