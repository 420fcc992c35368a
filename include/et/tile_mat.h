// 16x16 block-sparse weight container — the reference's tile_mat
// (mat_type/tile_mat/tile_mat.h:3-58): BSR over the [out x in] weight,
//   row_ptr[blk_row_num + 1], row_offset[num_blk] (column-tile index of every
//   tile, any order inside a block-row), data[num_blk * 256] (tile row-major,
//   tile rows = output features),
// all three resident on the device.  The layout is consumed unchanged by the
// MFMA kernel behind Linear<tile_mat>.
#pragma once
#include <utility>
#include <vector>

#include "CUDA_ptr.hpp"
#include "format_gen.h"

class tile_mat {
  public:
    static constexpr int tile_m = 16, tile_n = 16, tile_k = 16;
    static constexpr int tile_size = tile_m * tile_k;

    int blk_row_num;
    int blk_col_num;
    int num_blk;
    et::DeviceBuffer<int> row_ptr;
    et::DeviceBuffer<int> row_offset;
    et::DeviceBuffer<half> data;

    // host arrays -> device; the tile data is left zero (tile_mat.h:17-25)
    tile_mat(int _blk_row_num, int _blk_col_num, int _num_blk, const int *_row_ptr,
             const int *_row_offset, const half *_data)
        : blk_row_num(_blk_row_num), blk_col_num(_blk_col_num), num_blk(_num_blk),
          row_ptr(_row_ptr, (std::size_t)_blk_row_num + 1), row_offset(_row_offset, (std::size_t)_num_blk),
          data((std::size_t)_num_blk * tile_size) {
        if (_data) data = et::DeviceBuffer<half>(_data, (std::size_t)_num_blk * tile_size);
    }
    // deep copies of device buffers (tile_mat.h:26-35)
    tile_mat(const et::DeviceBuffer<int> &_row_ptr, const et::DeviceBuffer<int> &_row_offset,
             const et::DeviceBuffer<half> &_data, int _blk_col_num)
        : blk_row_num((int)_row_ptr.size - 1), blk_col_num(_blk_col_num),
          num_blk((int)(_data.size / tile_size)), row_ptr(_row_ptr), row_offset(_row_offset), data(_data) {}
    // host vectors, validated (tile_mat.h:36-45) — the loader path
    tile_mat(const std::vector<int> &_row_ptr, const std::vector<int> &_row_offset,
             const std::vector<half> &_data, int _blk_col_num)
        : blk_row_num((int)_row_ptr.size() - 1), blk_col_num(_blk_col_num),
          num_blk((int)(_data.size() / tile_size)), row_ptr(_row_ptr), row_offset(_row_offset), data(_data) {
        et::fmt::validate_bsr16(_row_ptr, _row_offset, _data.size() / tile_size, _blk_col_num);
    }
    // buffers moved in (tile_mat.h:46-55)
    tile_mat(et::DeviceBuffer<int> &&_row_ptr, et::DeviceBuffer<int> &&_row_offset,
             et::DeviceBuffer<half> &&_data, int _blk_col_num)
        : blk_row_num((int)_row_ptr.size - 1), blk_col_num(_blk_col_num),
          num_blk((int)(_data.size / tile_size)), row_ptr(std::move(_row_ptr)),
          row_offset(std::move(_row_offset)), data(std::move(_data)) {}

    int nrow() const { return blk_row_num * tile_m; }
    int ncol() const { return blk_col_num * tile_k; }

    // Random structure, all values 1.0 (mat_type/tile_mat/tile_mat.cu:7-40);
    // the shuffle is the seeded permutation of format_gen.h.
    static tile_mat gen_sparse_mat(int nrow, int ncol, float sparsity,
                                   uint64_t seed = et::fmt::kDefaultSeed) {
        auto p = et::fmt::gen_tile_pattern(nrow, ncol, sparsity, seed);
        et::DeviceBuffer<half> values(p.row_offset.size() * tile_size, half_one);
        return tile_mat(et::DeviceBuffer<int>(p.row_ptr), et::DeviceBuffer<int>(p.row_offset),
                        std::move(values), ncol / tile_k);
    }
    // Every tile present, all values 1.0 (mat_type/tile_mat/tile_mat.cu:42-64).
    static tile_mat gen_dense_mat(int nrow, int ncol) {
        auto p = et::fmt::dense_tile_pattern(nrow, ncol);
        et::DeviceBuffer<half> values(p.row_offset.size() * tile_size, half_one);
        return tile_mat(et::DeviceBuffer<int>(p.row_ptr), et::DeviceBuffer<int>(p.row_offset),
                        std::move(values), ncol / tile_k);
    }
    // BSR of a dense fp32 [nrow x ncol] host matrix with the exporter's rule
    // (example/npy2pt.py:75-109), values rounded to fp16 (round-to-nearest-even).
    static tile_mat from_dense(const float *W, int nrow, int ncol) {
        auto m = et::fmt::dense_to_bsr16(W, nrow, ncol);
        std::vector<half> h(m.data.size());
        for (std::size_t i = 0; i < h.size(); i++) h[i] = static_cast<half>(m.data[i]);
        return tile_mat(m.row_ptr, m.column, h, ncol / tile_k);
    }
};
