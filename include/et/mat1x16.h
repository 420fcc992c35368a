// 1x16 vector-sparse weight — the reference's mat1x16 (mat_type/mat1x16/mat1x16.h:5-22)
// in the layout its kernel reads (Linear/SPMM1x16.cu:52-74): for row-set r
// (16 output rows) and part p (16 input columns) the live 1x16 vectors are
// idx in [tile_idx[r*(npart+1)+p], tile_idx[r*(npart+1)+p+1]); row_idx[idx] % 16
// is the row inside the set, data[16*idx .. 16*idx+15] the weights.
#pragma once
#include <vector>

#include "CUDA_ptr.hpp"
#include "format_gen.h"

class mat1x16 {
  public:
    const int npart;
    const int nrow;
    const int ncol;
    const int ntile;
    et::DeviceBuffer<int> tile_idx;  // (nrow/16) * (npart + 1)
    et::DeviceBuffer<int> row_idx;   // ntile
    et::DeviceBuffer<half> data;     // pad16(ntile) * 16

    mat1x16(int _nrow, int _ncol, const std::vector<int> &_tile_idx, const std::vector<int> &_row_idx,
            const std::vector<half> &_data)
        : npart(_ncol / 16), nrow(_nrow), ncol(_ncol), ntile((int)_row_idx.size()), tile_idx(_tile_idx),
          row_idx(_row_idx), data(_data) {
        et::require(_tile_idx.size() == (std::size_t)(_nrow / 16) * (std::size_t)(npart + 1),
                    "mat1x16: tile_idx must hold (nrow/16)*(ncol/16+1) offsets");
        et::require(_tile_idx.empty() || _tile_idx.back() == ntile, "mat1x16: tile_idx must end at ntile");
        et::require(_data.size() >= (std::size_t)ntile * 16, "mat1x16: data shorter than ntile*16");
    }

    static mat1x16 from_parts(int nrow, int ncol, const et::fmt::Vec1x16 &m, half fill) {
        const std::size_t padded = ((m.row_idx.size() + 15) / 16) * 16 * 16;
        std::vector<half> h(padded, fill);
        for (std::size_t i = 0; i < m.data.size() && i < padded; i++) h[i] = static_cast<half>(m.data[i]);
        return mat1x16(nrow, ncol, m.tile_idx, m.row_idx, h);
    }
    // every vector present, values 1.0 (intent of mat_type/mat1x16/mat1x16.cu:15-36)
    static mat1x16 gen_dense_mat(int nrow, int ncol) {
        std::vector<float> ones((std::size_t)nrow * ncol, 1.0f);
        return from_parts(nrow, ncol, et::fmt::dense_to_1x16(ones.data(), nrow, ncol), half_one);
    }
    // seeded random vectors, values 1.0 (intent of mat_type/mat1x16/mat1x16.cu:38-75)
    static mat1x16 gen_sparse_mat(int nrow, int ncol, float sparsity,
                                  uint64_t seed = et::fmt::kDefaultSeed) {
        return from_parts(nrow, ncol, et::fmt::gen_1x16_pattern(nrow, ncol, sparsity, seed), half_one);
    }
    static mat1x16 from_dense(const float *W, int nrow, int ncol) {
        return from_parts(nrow, ncol, et::fmt::dense_to_1x16(W, nrow, ncol), half_zero);
    }
};
