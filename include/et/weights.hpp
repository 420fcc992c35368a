// Model weight loader with the reference's interface (example/weights.hpp:11-48):
// `filename` lists one archive name per line (weights.txt), each archive
// `path + name` is an .npz written by the exporter (example/npy2pt.py:112-119):
//   2-D weight: row_ptr int32[out/16+1], column int32[ntile],
//               data float32[ntile,256], B float32[out]
//   1-D weight: W float32[H], B float32[H]
#pragma once
#include <fstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "half.h"
#include "npy.hpp"

class Weights {
  public:
    std::vector<std::string> layer_names;
    std::string path;
    std::unordered_map<std::string, et::npy::npz_t> weight_files;

    Weights(const std::string &filename, const std::string &_path) : path(_path) {
        std::ifstream fin(filename);
        if (!fin) throw et::Error(ET_ERR_IO, "cannot open " + filename);
        std::string line;
        while (std::getline(fin, line)) {
            while (!line.empty() && (line.back() == '\r' || line.back() == ' ')) line.pop_back();
            if (!line.empty()) layer_names.push_back(line);
        }
        for (const auto &name : layer_names) weight_files.emplace(name, et::npy::npz_load(path + name));
    }

    bool has(const std::string &name, const std::string &npz_name) const {
        auto f = weight_files.find(npz_name);
        return f != weight_files.end() && f->second.count(name) != 0;
    }

    template <typename T> std::vector<T> load_mat(const std::string &name, const std::string &npz_name) const {
        auto f = weight_files.find(npz_name);
        if (f == weight_files.end()) throw et::Error(ET_ERR_IO, "no archive named " + npz_name);
        auto a = f->second.find(name);
        if (a == f->second.end()) throw et::Error(ET_ERR_IO, npz_name + " holds no array " + name);
        return a->second.as_vector<T>();
    }
};

// fp32 -> fp16, round-to-nearest-even (example/main.cu:195-200)
inline std::vector<half> vec_F2H(const std::vector<float> &arr) {
    std::vector<half> res(arr.size());
    for (std::size_t i = 0; i < arr.size(); i++) res[i] = static_cast<half>(arr[i]);
    return res;
}
