// The pre-multiplied value/output projection of the E.T. fused attention — the
// reference's Linear_VO / Linear_VO_prune (Fused_attention/Linear_VO.h:22-96):
//   VO[b][h] (S x N) = X[b] (S x H) * W[h] (H x N) + bias[h]
// with W "fully pre-processed": W[h] = W_V,h^T * W_O[:, h]^T, row-major [nh][H][N]
// (build_vo_weight below constructs it; the reference assumes it is made offline).
// One strided-batched MFMA GEMM with the per-head bias in its epilogue.  The
// result is laid out [batch][nh][S][N] — for batch 1 the reference's [nh][S][N].
#pragma once
#include <memory>
#include <vector>

#include "CUDA_ptr.hpp"
#include "Model.h"
#include "col_mat.hpp"

namespace et {
// Wt: the weights k-contiguous per head, [nh][N][H] (transposed_heads below)
inline void linear_vo_forward(const half *Wt, const half *bias, const half *X, half *out, const Model_t &m,
                              int batch, int N, stream_t stream) {
    etChk(et_linear_vo_t_f16(reinterpret_cast<const et_f16 *>(Wt), reinterpret_cast<const et_f16 *>(bias),
                             reinterpret_cast<const et_f16 *>(X), reinterpret_cast<et_f16 *>(out), batch,
                             m.seq_len, m.emdim, N, m.nhead, stream));
}

// The projection key-contiguous and without its bias, [batch][nh][N][S]: the operand layout of the
// attention kernel that keeps the probabilities on chip (et_mha_vo_otf_f16 adds the bias itself).
inline void linear_vo_forward_keys(const half *Wt, const half *X, half *out, const Model_t &m, int batch, int N,
                                   stream_t stream) {
    etChk(et_linear_vo_keys_f16(reinterpret_cast<const et_f16 *>(Wt), reinterpret_cast<const et_f16 *>(X),
                                reinterpret_cast<et_f16 *>(out), batch, m.seq_len, m.emdim, N, m.nhead, stream));
}

// Device copy of W[nh][H][N] turned into [nh][N][H], made once at construction: the GEMM behind
// the projection reads k-contiguous operands about twice as fast.
inline DeviceBuffer<half> transposed_heads(const half *W_dev, int nhead, int H, int N) {
    DeviceBuffer<half> t((std::size_t)nhead * H * N);
    etChk(et_transpose_heads_f16(reinterpret_cast<et_f16 *>(t.get()), reinterpret_cast<const et_f16 *>(W_dev), nhead,
                                 H, N, nullptr));
    etChk(et_device_sync());
    return t;
}

// W_VO[h] = W_V[h*hd:(h+1)*hd, :]^T * W_O[:, h*hd:(h+1)*hd]^T   ([H x N], N = emdim)
// b_VO[h] = b_V[h*hd:(h+1)*hd] * W_O[:, h*hd:(h+1)*hd]^T
// from host fp32 W_V [vdim x H], W_O [N x vdim].  Outputs sized nh*H*N and nh*N.
inline void build_vo_weight(const float *Wv, const float *bv, const float *Wo, int H, int vdim, int N,
                            int nhead, std::vector<float> &Wvo, std::vector<float> &bvo) {
    const int hd = vdim / nhead;
    Wvo.assign((std::size_t)nhead * H * N, 0.0f);
    bvo.assign((std::size_t)nhead * N, 0.0f);
    for (int h = 0; h < nhead; h++)
        for (int d = 0; d < hd; d++) {
            const int f = h * hd + d;  // V feature
            for (int n = 0; n < N; n++) {
                const float wo = Wo[(std::size_t)n * vdim + f];
                if (wo == 0.0f) continue;
                if (bv) bvo[(std::size_t)h * N + n] += bv[f] * wo;
                float *dst = &Wvo[((std::size_t)h * H) * N + n];
                const float *src = &Wv[(std::size_t)f * H];
                for (int i = 0; i < H; i++) dst[(std::size_t)i * N] += src[i] * wo;
            }
        }
}
}  // namespace et

class Linear_VO {
    using ptr_t = et::DeviceBuffer<half>;

  public:
    ptr_t bias;    // [nh][N]
    ptr_t weight;  // [nh][H][N] row-major
    std::shared_ptr<Model_t> model;
    ptr_t weight_t;  // [nh][N][H]: what forward() reads

    Linear_VO(const ptr_t &_weight, const ptr_t &_bias, std::shared_ptr<Model_t> _model)
        : bias(_bias), weight(_weight), model(std::move(_model)),
          weight_t(checked_transpose(weight, *model)) {
        et::require(bias.size == (std::size_t)model->nhead * model->emdim, "Linear_VO: bias must be [nhead][emdim]");
    }
    int out_width() const { return model->emdim; }
    void forward(half *output, const half *input, et::stream_t stream = nullptr, int batch = 1) {
        et::linear_vo_forward(weight_t.get(), bias.get(), input, output, *model, batch, model->emdim, stream);
    }
    void forward_keys(half *output, const half *input, et::stream_t stream = nullptr, int batch = 1) {
        et::linear_vo_forward_keys(weight_t.get(), input, output, *model, batch, model->emdim, stream);
    }

  private:
    static ptr_t checked_transpose(const ptr_t &w, const Model_t &m) {
        et::require(w.size == (std::size_t)m.nhead * m.emdim * m.emdim, "Linear_VO: weight must be [nhead][emdim][emdim]");
        return et::transposed_heads(w.get(), m.nhead, m.emdim, m.emdim);
    }
};

// Column-pruned W_VO: only the output columns col_id survive; weight.cols is
// [nh][H][len(col_id)], bias [nh][len(col_id)] (Fused_attention/Linear_VO.h:61-96).
class Linear_VO_prune {
    using ptr_t = et::DeviceBuffer<half>;

  public:
    ptr_t bias;
    col_mat weight;
    std::shared_ptr<Model_t> model;
    ptr_t weight_t;  // [nh][len(col_id)][H]: what forward() reads

    Linear_VO_prune(const col_mat &_weight, const ptr_t &_bias, std::shared_ptr<Model_t> _model)
        : bias(_bias), weight(_weight), model(std::move(_model)), weight_t(checked_transpose(weight, *model)) {
        et::require(bias.size == (std::size_t)model->nhead * weight.col_id->size,
                    "Linear_VO_prune: bias must be [nhead][len(col_id)]");
    }
    int out_width() const { return (int)weight.col_id->size; }
    void forward(half *output, const half *input, et::stream_t stream = nullptr, int batch = 1) {
        et::linear_vo_forward(weight_t.get(), bias.get(), input, output, *model, batch, out_width(), stream);
    }
    void forward_keys(half *output, const half *input, et::stream_t stream = nullptr, int batch = 1) {
        et::linear_vo_forward_keys(weight_t.get(), input, output, *model, batch, out_width(), stream);
    }

  private:
    static ptr_t checked_transpose(const col_mat &w, const Model_t &m) {
        const std::size_t n = w.col_id->size;
        et::require(w.cols->size == (std::size_t)m.nhead * m.emdim * n,
                    "Linear_VO_prune: weight must be [nhead][emdim][len(col_id)]");
        return et::transposed_heads(w.cols->get(), m.nhead, m.emdim, (int)n);
    }
};
