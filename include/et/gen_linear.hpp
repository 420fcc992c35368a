// Test-data Linear factories with the reference's conventions
// (Linear/gen_linear.hpp:1-27, Linear/Linear.cu:7-22): nrow = out features,
// ncol = in features, every weight value 1.0 (0.5 for col_mat), bias 0.5.
#pragma once
#include <memory>
#include <vector>

template <typename T> std::unique_ptr<Linear<T>> gen_dense_linear(int nrow, int ncol, int size) {
    std::vector<half> bias((std::size_t)nrow, static_cast<half>(0.5f));
    return std::make_unique<Linear<T>>(ncol, nrow, T::gen_dense_mat(nrow, ncol), bias.data(), size);
}

template <>
inline std::unique_ptr<Linear<base_mat>> gen_dense_linear<base_mat>(int nrow, int ncol, int size) {
    std::vector<half> bias((std::size_t)nrow, static_cast<half>(0.5f));
    return std::make_unique<Linear<base_mat>>(ncol, nrow, base_mat((std::size_t)nrow * ncol, half_one),
                                              bias.data(), size);
}

template <typename T>
std::unique_ptr<Linear<T>> gen_sparse_linear(int nrow, int ncol, int size, float sparsity) {
    std::vector<half> bias((std::size_t)nrow, static_cast<half>(0.5f));
    return std::make_unique<Linear<T>>(ncol, nrow, T::gen_sparse_mat(nrow, ncol, sparsity), bias.data(), size);
}

// a dense weight has no sparse form: same as gen_dense_linear (Linear/Linear.cu:17-22)
template <>
inline std::unique_ptr<Linear<base_mat>> gen_sparse_linear<base_mat>(int nrow, int ncol, int size, float) {
    return gen_dense_linear<base_mat>(nrow, ncol, size);
}
