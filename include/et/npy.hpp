// Reader for NumPy .npy arrays and .npz archives (zip of .npy, stored or
// deflated) — what the reference obtains from the un-vendored cnpy library
// (example/weights.hpp:4,45).  Implemented in scpaper-2021_amd/host/npz.cpp.
#pragma once
#include <cstddef>
#include <map>
#include <string>
#include <vector>

#include "status.h"

namespace et {
namespace npy {

struct Array {
    std::string descr;               // e.g. "<f4", "<i4"
    std::vector<std::size_t> shape;
    std::size_t word_size = 0;       // bytes per element
    bool fortran_order = false;
    std::vector<char> bytes;

    std::size_t num_vals() const {
        std::size_t n = 1;
        for (std::size_t d : shape) n *= d;
        return n;
    }
    template <typename T> const T *data() const { return reinterpret_cast<const T *>(bytes.data()); }
    // element-typed copy; throws if the element size does not match
    template <typename T> std::vector<T> as_vector() const {
        if (word_size != sizeof(T)) throw Error(ET_ERR_IO, "npy: element size mismatch for descr " + descr);
        return std::vector<T>(data<T>(), data<T>() + num_vals());
    }
};

using npz_t = std::map<std::string, Array>;  // keyed by array name (without ".npy")

Array parse_npy(const char *buf, std::size_t len, const std::string &what);
// writes a little-endian C-order .npy (version 1.0); descr e.g. "<f4", "<i4", "<f2"
void npy_save(const std::string &path, const void *data, const std::string &descr, std::size_t word_size,
              const std::vector<std::size_t> &shape);
Array npy_load(const std::string &path);
npz_t npz_load(const std::string &path);

}  // namespace npy
}  // namespace et
