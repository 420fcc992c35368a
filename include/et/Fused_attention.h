// Attention with the pre-computed VO projection — the reference's
// FusedAttention<cfg> (Fused_attention/Fused_attention.h:34-118):
//   VO_h = X W_VO,h + b_VO,h          (Linear_VO)
//   out  = sum_h softmax(Q_h K_h^T / sqrt(hd) + mask) VO_h + b_O
// OTF_fused_attn keeps the probabilities on chip (Fused_attention/Fused_attention.cu:10-116):
// the projection is written key-contiguous, the waves of a workgroup take a head each.
// The NOTF tags write P once as [rows x nh*S] (Fused_attention/Fused_attention.cu:
// 201-204) and run ONE MFMA GEMM per sequence, [S x nh*S] * [nh*S x N].  Both add
// b_O — and, for the pruned form, scatter the N surviving columns to full width —
// in the epilogue, accumulate in fp32 and write every output element exactly once,
// where the reference's OTF kernel adds fp16 atomics into an output it never clears.
#pragma once
#include <memory>
#include <type_traits>

#include "Attention.h"
#include "Linear_VO.h"

struct OTF_fused_attn {};
struct NOTF_fused_attn {};
struct NOTF_fused_prune_attn {};

template <typename T> struct __VO_helper { using type = Linear_VO; };
template <> struct __VO_helper<NOTF_fused_prune_attn> { using type = Linear_VO_prune; };

template <typename _config> class FusedAttention : public et::AttnState {
    using ptr_t = et::DeviceBuffer<half>;
    using config = _config;
    using linearQ_t = Linear<typename config::WQ_t>;
    using linearK_t = Linear<typename config::WK_t>;
    using LinearVO_t = typename __VO_helper<typename config::attn_t>::type;
    static constexpr bool kPruned = std::is_same<typename config::attn_t, NOTF_fused_prune_attn>::value;
    static constexpr bool kOnChip = std::is_same<typename config::attn_t, OTF_fused_attn>::value;

    std::unique_ptr<linearQ_t> linearQ;
    std::unique_ptr<linearK_t> linearK;
    std::unique_ptr<LinearVO_t> linearVO;
    ptr_t biasO;
    std::unique_ptr<ptr_t> mat_k, mat_q, mat_qk, mat_vo;
    std::shared_ptr<Model_t> model;

  public:
    FusedAttention(std::unique_ptr<linearQ_t> _linearQ, std::unique_ptr<linearK_t> _linearK,
                   std::unique_ptr<LinearVO_t> _linearVO, const ptr_t &_biasO, std::shared_ptr<Model_t> _model,
                   int batch = 1)
        : et::AttnState(_model, batch), linearQ(std::move(_linearQ)), linearK(std::move(_linearK)),
          linearVO(std::move(_linearVO)), biasO(_biasO), model(_model) {
        const std::size_t T = (std::size_t)rows();
        mat_k = std::make_unique<ptr_t>(T * model->kdim);
        mat_q = std::make_unique<ptr_t>(T * model->kdim);
        if (!kOnChip) mat_qk = std::make_unique<ptr_t>(T * model->seq_len * model->nhead);
        mat_vo = std::make_unique<ptr_t>(T * model->nhead * (std::size_t)linearVO->out_width());
        et::require(biasO.size == (std::size_t)model->emdim, "FusedAttention: biasO must hold emdim values");
    }

    void forward(half *out, half *query, half *key, half *value, et::stream_t stream = nullptr) {
        if constexpr (kOnChip) linearVO->forward_keys(mat_vo->get(), value, stream, batch());
        else linearVO->forward(mat_vo->get(), value, stream, batch());
        linearQ->forward(mat_q->get(), query, stream);
        linearK->forward(mat_k->get(), key, stream);
        const et::AttnRun r = run(stream);
        const int hd = model->kdim / model->nhead;
        const float scale = 1.0f / std::sqrt((float)hd);
        const int *scatter = nullptr;
        if constexpr (kPruned) scatter = linearVO->weight.col_id->get();
        if constexpr (kOnChip) {
            etChk(et_mha_vo_otf_f16(et::f16(mat_q->get()), et::f16(mat_k->get()), model->kdim, model->kdim,
                                    et::f16(mat_vo->get()), et::f16(linearVO->bias.get()), et::f16(out),
                                    et::f16(biasO.get()), scatter,
                                    et::f16(r.mask), r.lens, r.batch, model->seq_len, model->nhead, hd,
                                    linearVO->out_width(), model->emdim, scale, r.causal ? ET_MHA_CAUSAL : 0, stream));
            return;
        }
        etChk(et_mha_vo_f16(et::f16(mat_q->get()), et::f16(mat_k->get()), model->kdim, model->kdim,
                            et::f16(mat_vo->get()), et::f16(mat_qk->get()), et::f16(out), et::f16(biasO.get()),
                            scatter, et::f16(r.mask), r.lens, r.batch, model->seq_len, model->nhead, hd,
                            linearVO->out_width(), model->emdim, scale, r.causal ? ET_MHA_CAUSAL : 0, stream));
    }
};
