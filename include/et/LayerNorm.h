// out = LayerNorm(src) * weight + bias — the reference's LayerNorm
// (LayerNorm/LayerNorm.h:6-16), eps 1e-5 (LayerNorm/LayerNorm.cu:37-38).  One pass
// over memory and no device synchronisation (the reference makes three passes and
// blocks the host, LayerNorm/LayerNorm.cu:51-57).
#pragma once
#include <memory>
#include <vector>

#include "CUDA_ptr.hpp"

class LayerNorm {
    const float eps;
    const int size;
    et::DeviceBuffer<half> weight;
    et::DeviceBuffer<half> bias;

  public:
    LayerNorm(const half *w, const half *b, int _size, float _eps = 1e-5f)
        : eps(_eps), size(_size), weight(w, (std::size_t)_size), bias(b, (std::size_t)_size) {}
    void forward(half *out, const half *src, int num, et::stream_t stream = nullptr) const {
        etChk(et_layernorm_f16(reinterpret_cast<et_f16 *>(out), reinterpret_cast<const et_f16 *>(src),
                               reinterpret_cast<const et_f16 *>(weight.get()),
                               reinterpret_cast<const et_f16 *>(bias.get()), num, size, eps, stream));
    }
};

// gamma = beta = 0.2 (LayerNorm/LayerNorm.cu:59-63)
inline std::unique_ptr<LayerNorm> gen_LN(int size) {
    std::vector<half> w((std::size_t)size, static_cast<half>(0.2f)), b((std::size_t)size, static_cast<half>(0.2f));
    return std::make_unique<LayerNorm>(w.data(), b.data(), size);
}
