// Input-feature ("column of W") pruned weight — the reference's col_mat
// (mat_type/col_mat/col_mat.hpp:10-73): cols[nrow x nnz_col] row-major holds the
// surviving columns of the [nrow x ncol] = [out x in] weight, col_id[nnz_col]
// their positions (any order).  The same container doubles as the compact V
// activation of the attention-aware path: [seq rows x surviving V columns] with
// head_ptr[nhead + 1] delimiting each head's columns (set_metadata).
#pragma once
#include <fstream>
#include <memory>
#include <string>
#include <vector>

#include "CUDA_ptr.hpp"
#include "format_gen.h"

class col_mat {
  public:
    int nrow = 0;
    int ncol = 0;
    int nnz_col = 0;
    int ldm = 0;  // row stride of cols
    std::unique_ptr<et::DeviceBuffer<int>> head_ptr;
    std::unique_ptr<et::DeviceBuffer<int>> col_id;
    std::unique_ptr<et::DeviceBuffer<half>> cols;
    std::vector<int> head_ptr_host;  // host copy of head_ptr (empty until set_metadata)

    // file: i32 nrow, ncol, len_id; i32 col_id[len_id]; f32 cols[nrow*len_id]
    // (mat_type/col_mat/col_mat.hpp:22-36)
    explicit col_mat(const std::string &filename) {
        std::ifstream f(filename, std::ios::binary);
        if (!f) throw et::Error(ET_ERR_IO, "cannot open " + filename);
        int32_t meta[3];
        f.read(reinterpret_cast<char *>(meta), sizeof meta);
        if (!f) throw et::Error(ET_ERR_IO, filename + ": truncated header");
        nrow = meta[0];
        ncol = meta[1];
        nnz_col = meta[2];
        f.seekg(0, std::ios::end);
        const std::size_t file_bytes = (std::size_t)f.tellg();
        f.seekg(12, std::ios::beg);
        if (nrow <= 0 || ncol <= 0 || nnz_col < 0 || nnz_col > ncol || file_bytes < 12 + 4 * (std::size_t)nnz_col ||
            (nnz_col > 0 && (file_bytes - 12 - 4 * (std::size_t)nnz_col) / 4 / (std::size_t)nnz_col < (std::size_t)nrow))
            throw et::Error(ET_ERR_IO, filename + ": header does not match the file size");
        std::vector<int> ids((std::size_t)nnz_col);
        std::vector<float> vals((std::size_t)nrow * nnz_col);
        f.read(reinterpret_cast<char *>(ids.data()), (std::streamsize)(ids.size() * 4));
        f.read(reinterpret_cast<char *>(vals.data()), (std::streamsize)(vals.size() * 4));
        if (!f) throw et::Error(ET_ERR_IO, filename + ": truncated");
        for (int id : ids)
            if (id < 0 || id >= ncol) throw et::Error(ET_ERR_IO, filename + ": column id outside the matrix");
        std::vector<half> h(vals.size());
        for (std::size_t i = 0; i < h.size(); i++) h[i] = static_cast<half>(vals[i]);
        col_id = std::make_unique<et::DeviceBuffer<int>>(ids);
        cols = std::make_unique<et::DeviceBuffer<half>>(h);
        ldm = nnz_col;
    }
    col_mat(const et::DeviceBuffer<int> &_col_id, const et::DeviceBuffer<half> &_cols, int _nrow, int _ncol,
            int _nnz_col)
        : nrow(_nrow), ncol(_ncol), nnz_col(_nnz_col),
          col_id(std::make_unique<et::DeviceBuffer<int>>(_col_id)),
          cols(std::make_unique<et::DeviceBuffer<half>>(_cols)) {
        ldm = _nrow ? (int)(cols->size / (std::size_t)_nrow) : 0;
    }
    col_mat(et::DeviceBuffer<int> &&_col_id, et::DeviceBuffer<half> &&_cols, int _nrow, int _ncol, int _nnz_col)
        : nrow(_nrow), ncol(_ncol), nnz_col(_nnz_col),
          col_id(std::make_unique<et::DeviceBuffer<int>>(std::move(_col_id))),
          cols(std::make_unique<et::DeviceBuffer<half>>(std::move(_cols))) {
        ldm = _nrow ? (int)(cols->size / (std::size_t)_nrow) : 0;
    }
    // Copies carry every field (the reference's leave nrow/ncol/nnz_col unset).
    col_mat(const col_mat &m)
        : nrow(m.nrow), ncol(m.ncol), nnz_col(m.nnz_col), ldm(m.ldm), head_ptr_host(m.head_ptr_host) {
        if (m.head_ptr) head_ptr = std::make_unique<et::DeviceBuffer<int>>(*m.head_ptr);
        col_id = std::make_unique<et::DeviceBuffer<int>>(*m.col_id);
        cols = std::make_unique<et::DeviceBuffer<half>>(*m.cols);
    }
    col_mat(col_mat &&m) noexcept = default;
    // empty container of a given shape (col_mat.hpp:64-69): the compact V buffer
    col_mat(int _nrow, int _ncol, int _nn_col)
        : nrow(_nrow), ncol(_ncol), nnz_col(_nn_col), ldm(_nn_col),
          col_id(std::make_unique<et::DeviceBuffer<int>>((std::size_t)_nn_col)),
          cols(std::make_unique<et::DeviceBuffer<half>>((std::size_t)_nrow * _nn_col)) {}

    col_mat *get() { return this; }

    // Records which full-width columns the compact columns stand for and splits
    // them by head (mat_type/col_mat/col_mat.cu:34-58).  _col_id must be ascending.
    void set_metadata(const et::DeviceBuffer<int> &_col_id, int _nnz_col, int nhead, int full_dim) {
        std::vector<int> ids = _col_id.to_host();
        head_ptr_host = et::fmt::head_ptr(ids, _nnz_col, nhead, full_dim);
        nnz_col = _nnz_col;
        head_ptr = std::make_unique<et::DeviceBuffer<int>>(head_ptr_host);
        col_id = std::make_unique<et::DeviceBuffer<int>>(_col_id);
    }

    // every column kept, values 1.0 (mat_type/col_mat/col_mat.cu:14-20)
    static col_mat gen_dense_mat(int nrow, int ncol) {
        std::vector<int> ids((std::size_t)ncol);
        for (int i = 0; i < ncol; i++) ids[(std::size_t)i] = i;
        return col_mat(et::DeviceBuffer<int>(ids),
                       et::DeviceBuffer<half>((std::size_t)nrow * ncol, half_one), nrow, ncol, ncol);
    }
    // kept-column count rounded down to a multiple of 16, ids in permuted order,
    // values 0.5 (mat_type/col_mat/col_mat.cu:22-32)
    static col_mat gen_sparse_mat(int nrow, int ncol, float sparsity,
                                  uint64_t seed = et::fmt::kDefaultSeed) {
        auto ids = et::fmt::gen_col_ids(ncol, sparsity, seed);
        const int nn = (int)ids.size();
        et::DeviceBuffer<half> values((std::size_t)nrow * nn, static_cast<half>(0.5f));
        return col_mat(et::DeviceBuffer<int>(ids), std::move(values), nrow, ncol, nn);
    }
};
