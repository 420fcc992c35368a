// Unstructured CSR weight on the host — the reference's csr_mat
// (mat_type/csr_mat/csr_mat.h:11-42); Linear<csr_mat> uploads it.
#pragma once
#include <string>
#include <vector>

#include "format_gen.h"

struct csr_mat {
    std::vector<int> indptr;
    std::vector<int> indices;
    std::vector<float> data;
    int nrow;
    int ncol;
    int nnz;

    csr_mat() = delete;
    // .csr file: u32 nrow, ncol, nnz; i32 indptr[nrow+1]; i32 indices[nnz]; f32 data[nnz]
    explicit csr_mat(const std::string &path) : csr_mat(et::fmt::read_csr(path)) {}
    csr_mat(std::vector<int> _indptr, std::vector<int> _indices, std::vector<float> _data, int _nrow,
            int _ncol, int _nnz)
        : indptr(std::move(_indptr)), indices(std::move(_indices)), data(std::move(_data)), nrow(_nrow),
          ncol(_ncol), nnz(_nnz) {}
    explicit csr_mat(et::fmt::Csr m)
        : indptr(std::move(m.indptr)), indices(std::move(m.indices)), data(std::move(m.data)),
          nrow(m.nrow), ncol(m.ncol), nnz(m.nnz) {}

    // all entries present, values 1.0 (mat_type/csr_mat/csr_mat.cpp:7-23)
    static csr_mat gen_dense_mat(int nrow, int ncol) {
        std::vector<float> ones((std::size_t)nrow * ncol, 1.0f);
        return csr_mat(et::fmt::dense_to_csr(ones.data(), nrow, ncol));
    }
    // seeded random entries, values 1.0 (mat_type/csr_mat/csr_mat.cpp:25-67)
    static csr_mat gen_sparse_mat(int nrow, int ncol, float sparsity,
                                  uint64_t seed = et::fmt::kDefaultSeed) {
        return csr_mat(et::fmt::gen_csr_pattern(nrow, ncol, sparsity, seed));
    }
};
