// Output-feature ("row of W") pruned weight — the reference's row_mat
// (mat_type/row_mat/row_mat.hpp:9-56): rows[nnz_row x ncol] holds the surviving
// rows of the [nrow x ncol] = [out x in] weight, row_id[nnz_row] (ascending)
// their positions.
#pragma once
#include <fstream>
#include <memory>
#include <string>
#include <vector>

#include "CUDA_ptr.hpp"
#include "format_gen.h"

class row_mat {
  public:
    int nrow;
    int ncol;
    std::unique_ptr<et::DeviceBuffer<int>> row_id;
    std::unique_ptr<et::DeviceBuffer<half>> rows;

    // .row file: u32 nrow, ncol, len_id; i32 row_id[len_id]; f32 rows[len_id*ncol]
    // (writer mat_type/row_mat/gen_mat.py:17-29, reader row_mat.hpp:15-29)
    explicit row_mat(const std::string &filename) {
        std::ifstream f(filename, std::ios::binary);
        if (!f) throw et::Error(ET_ERR_IO, "cannot open " + filename);
        uint32_t meta[3];
        f.read(reinterpret_cast<char *>(meta), sizeof meta);
        if (!f) throw et::Error(ET_ERR_IO, filename + ": truncated header");
        nrow = (int)meta[0];
        ncol = (int)meta[1];
        const std::size_t len = meta[2];
        // the header must describe the file: counts that do not fit its size are refused before
        // anything is allocated from them
        f.seekg(0, std::ios::end);
        const std::size_t file_bytes = (std::size_t)f.tellg();
        f.seekg(12, std::ios::beg);
        if (nrow <= 0 || ncol <= 0 || len > (std::size_t)nrow ||
            file_bytes < 12 + 4 * len || (file_bytes - 12 - 4 * len) / 4 / (std::size_t)ncol < len)
            throw et::Error(ET_ERR_IO, filename + ": header does not match the file size");
        std::vector<int> ids(len);
        std::vector<float> vals(len * (std::size_t)ncol);
        f.read(reinterpret_cast<char *>(ids.data()), (std::streamsize)(ids.size() * 4));
        f.read(reinterpret_cast<char *>(vals.data()), (std::streamsize)(vals.size() * 4));
        if (!f) throw et::Error(ET_ERR_IO, filename + ": truncated");
        for (int id : ids)
            if (id < 0 || id >= nrow) throw et::Error(ET_ERR_IO, filename + ": row id outside the matrix");
        std::vector<half> h(vals.size());
        for (std::size_t i = 0; i < h.size(); i++) h[i] = static_cast<half>(vals[i]);
        row_id = std::make_unique<et::DeviceBuffer<int>>(ids);
        rows = std::make_unique<et::DeviceBuffer<half>>(h);
    }
    row_mat(const et::DeviceBuffer<int> &_row_id, const et::DeviceBuffer<half> &_rows, int _nrow, int _ncol)
        : nrow(_nrow), ncol(_ncol), row_id(std::make_unique<et::DeviceBuffer<int>>(_row_id)),
          rows(std::make_unique<et::DeviceBuffer<half>>(_rows)) {}
    row_mat(et::DeviceBuffer<int> &&_row_id, et::DeviceBuffer<half> &&_rows, int _nrow, int _ncol)
        : nrow(_nrow), ncol(_ncol), row_id(std::make_unique<et::DeviceBuffer<int>>(std::move(_row_id))),
          rows(std::make_unique<et::DeviceBuffer<half>>(std::move(_rows))) {}
    row_mat(const row_mat &m)
        : nrow(m.nrow), ncol(m.ncol), row_id(std::make_unique<et::DeviceBuffer<int>>(*m.row_id)),
          rows(std::make_unique<et::DeviceBuffer<half>>(*m.rows)) {}
    row_mat(row_mat &&m) noexcept = default;

    int nnz_row() const { return (int)row_id->size; }

    // every row kept, values 1.0 (mat_type/row_mat/row_mat.cu:5-12)
    static row_mat gen_dense_mat(int nrow, int ncol) {
        std::vector<int> ids((std::size_t)nrow);
        for (int i = 0; i < nrow; i++) ids[(std::size_t)i] = i;
        return row_mat(et::DeviceBuffer<int>(ids),
                       et::DeviceBuffer<half>((std::size_t)nrow * ncol, half_one), nrow, ncol);
    }
    // kept-row count padded up to a multiple of 16, ids ascending, values 1.0
    // (mat_type/row_mat/row_mat.cu:14-25)
    static row_mat gen_sparse_mat(int nrow, int ncol, float sparsity,
                                  uint64_t seed = et::fmt::kDefaultSeed) {
        auto ids = et::fmt::gen_row_ids(nrow, sparsity, seed);
        et::DeviceBuffer<half> values(ids.size() * (std::size_t)ncol, half_one);
        return row_mat(et::DeviceBuffer<int>(ids), std::move(values), nrow, ncol);
    }
};
