// out = LayerNorm(src + skip) * weight + bias over rows of `size` features — the
// reference's SkipLayerNorm (SkipLayerNorm/SkipLayerNorm.h:6-16), eps 1e-5
// (SkipLayerNorm/SkipLayerNorm.cu:70-71).  Statistics are fp32 and the variance
// is E[(x - mean)^2].
#pragma once
#include <memory>
#include <vector>

#include "CUDA_ptr.hpp"

class SkipLayerNorm {
    const float eps;
    const int size;
    et::DeviceBuffer<half> weight;
    et::DeviceBuffer<half> bias;

  public:
    // w, b: host pointers to `size` values
    SkipLayerNorm(const half *w, const half *b, int _size, float _eps = 1e-5f)
        : eps(_eps), size(_size), weight(w, (std::size_t)_size), bias(b, (std::size_t)_size) {}
    void forward(half *out, const half *src, const half *skip, int num, et::stream_t stream = nullptr) const {
        etChk(et_skip_layernorm_f16(reinterpret_cast<et_f16 *>(out), reinterpret_cast<const et_f16 *>(src),
                                    reinterpret_cast<const et_f16 *>(skip),
                                    reinterpret_cast<const et_f16 *>(weight.get()),
                                    reinterpret_cast<const et_f16 *>(bias.get()), num, size, eps, stream));
    }
    // mixed precision: src and skip binary32 (a projection's unrounded output and the residual
    // stream), result written as binary32 (out32, the next residual) and rounded to binary16
    // (out16, the next projection's operand); either output may be null
    void forward_mixed(float *out32, half *out16, const float *src, const float *skip, int num,
                       et::stream_t stream = nullptr) const {
        etChk(et_skip_layernorm_mixed(out32, reinterpret_cast<et_f16 *>(out16), src, skip,
                                      reinterpret_cast<const et_f16 *>(weight.get()),
                                      reinterpret_cast<const et_f16 *>(bias.get()), num, size, eps, stream));
    }
    int width() const { return size; }
    const half *gamma() const { return weight.get(); }
    const half *beta() const { return bias.get(); }
    float epsilon() const { return eps; }
};

// gamma = beta = 0.2, the reference's test instance (SkipLayerNorm/SkipLayerNorm.cu:84-88)
inline std::unique_ptr<SkipLayerNorm> gen_skLN(int size) {
    std::vector<half> w((std::size_t)size, static_cast<half>(0.2f)), b((std::size_t)size, static_cast<half>(0.2f));
    return std::make_unique<SkipLayerNorm>(w.data(), b.data(), size);
}
