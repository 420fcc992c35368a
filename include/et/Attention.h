// Multi-head self-attention block — the reference's Attention<cfg>
// (Attention/Attention.h:10-266): Q/K/V projections, fused attention, output
// projection, with the same configuration tags and constructor signatures.
//
// Differences from the reference, all deliberate:
//  * every on-the-fly tag runs the one fused gfx950 kernel (scores, mask,
//    softmax and P*V in registers/LDS, fp32 accumulation, 1/sqrt(hd) scale);
//    the tags stay distinct types so that callers keep compiling;
//  * a batch of sequences is supported: `batch` sequences of model->seq_len rows,
//    optional per-sequence key lengths (right padding);
//  * the mask is a property the caller sets (none by default, causal, or an
//    additive [S x S] matrix) instead of the hard-wired causal mask of
//    Attention/Attention.h:96-104;
//  * all launches go to ONE stream passed to forward(), nothing joins on the host
//    (the reference fans Q/K/V out to three streams and blocks on them,
//    Attention/Attention.h:122-127), so a forward can be captured into a HIP graph.
#pragma once
#include <cmath>
#include <memory>
#include <type_traits>
#include <vector>

#include "Linear.h"
#include "Model.h"

using ptr_t = et::DeviceBuffer<half>;

template <typename _WQ_t, typename _WK_t, typename _WV_t, typename _WO_t, typename _attn_t,
          bool _isSingleKernel = false, bool _isPara = true,
          typename = typename std::enable_if<!(_isSingleKernel && _isPara)>::type>
struct Attention_config {
    using WQ_t = _WQ_t;
    using WK_t = _WK_t;
    using WV_t = _WV_t;
    using WO_t = _WO_t;
    using attn_t = _attn_t;
    static constexpr bool isPara = _isPara;  // kept for source compatibility; one stream is used
    static constexpr bool isSingleKernel = _isSingleKernel;
    using W_t = typename std::conditional<_isSingleKernel, _WQ_t, void>::type;
};

// attention kernel tags (Attention/Attention.h:26-33)
struct OTF_attn {};
struct Norm_attn {};
struct Prune_attn {};
struct OTF_attn_full {};
struct OTF_attn_tile {};
struct OTF_attn_sharedQK {};
struct OTF_attn_full_mixed {};
struct OTF_attn_Ofused {};

namespace et {

// What a fused attention call needs beyond Q, K, V: sequences, mask, stream.
struct AttnRun {
    int batch = 1;
    const int *lens = nullptr;   // device int32[batch] or nullptr
    const half *mask = nullptr;  // device additive [S x S] or nullptr
    bool causal = false;
    float scale = 0.0f;          // 0 = 1/sqrt(head_dim)
    stream_t stream = nullptr;
    // Multihead_atttion_fuseO only: attention and output projection as ONE launch (et_mha_fuseo_f16), as the
    // reference runs them, instead of the two stream-ordered launches, which are several times faster here
    bool one_launch = false;
};

inline void fused_mha(const half *q, const half *k, const half *v, int ldq, int ldk, int ldv, half *z,
                      int ldz, const Model_t &m, const AttnRun &run) {
    const int hd = m.kdim / m.nhead;
    require(m.vdim == m.kdim, "fused attention: vdim must equal kdim");
    const float scale = run.scale != 0.0f ? run.scale : 1.0f / std::sqrt((float)hd);
    etChk(et_mha_fused_f16(f16(q), f16(k), f16(v), ldq, ldk, ldv, f16(z), ldz, f16(run.mask), run.lens,
                           run.batch, m.seq_len, m.nhead, hd, scale, run.causal ? ET_MHA_CAUSAL : 0,
                           run.stream));
}

}  // namespace et

// Free-function form (Attention/Attention.h:35-45,144-181).  mat_qk is unused by
// the fused kernel (scores never reach memory) and may be null.
template <typename _attn_type>
void Multihead_atttion(ptr_t *mat_q, ptr_t *mat_k, ptr_t *mat_v, ptr_t *mat_qk, const ptr_t *mask,
                       ptr_t *mat_z, std::shared_ptr<Model_t> model, et::AttnRun run = et::AttnRun()) {
    static_assert(!std::is_same<_attn_type, Prune_attn>::value, "Prune_attn takes a col_mat V");
    (void)mat_qk;
    if (mask && !run.mask) run.mask = mask->get();
    if constexpr (std::is_same<_attn_type, Norm_attn>::value) {
        // Unfused baseline: scores through memory (Attention/Attention.cu:8-36).
        et::require(mat_qk != nullptr, "Norm_attn needs the mat_qk workspace");
        const int hd = model->kdim / model->nhead;
        const float scale = run.scale != 0.0f ? run.scale : 1.0f / std::sqrt((float)hd);
        etChk(et_mha_unfused_f16(et::f16(mat_q->get()), et::f16(mat_k->get()), et::f16(mat_v->get()),
                                 model->kdim, model->kdim, model->vdim, et::f16(mat_z->get()), model->vdim,
                                 et::f16(mat_qk->get()), et::f16(run.mask), run.lens, run.batch,
                                 model->seq_len, model->nhead, hd, scale, run.causal ? ET_MHA_CAUSAL : 0,
                                 run.stream));
        return;
    }
    et::fused_mha(mat_q->get(), mat_k->get(), mat_v->get(), model->kdim, model->kdim, model->vdim,
                  mat_z->get(), model->vdim, *model, run);
}

// Attention-aware form: V is compact [S x nnz] with col_id / head_ptr metadata
// (Attention/Attention.cu:54-78).  Pruned columns of Z are written as zero.
template <typename _attn_type>
void Multihead_atttion(ptr_t *mat_q, ptr_t *mat_k, col_mat *mat_v, ptr_t *mat_qk, const ptr_t *mask,
                       ptr_t *mat_z, std::shared_ptr<Model_t> model, et::AttnRun run = et::AttnRun()) {
    static_assert(std::is_same<_attn_type, Prune_attn>::value, "a col_mat V belongs to Prune_attn");
    (void)mat_qk;
    if (mask && !run.mask) run.mask = mask->get();
    et::require(mat_v->head_ptr != nullptr, "Prune_attn: col_mat::set_metadata was not called");
    const int hd = model->kdim / model->nhead;
    const float scale = run.scale != 0.0f ? run.scale : 1.0f / std::sqrt((float)hd);
    etChk(et_mha_compactv_f16(et::f16(mat_q->get()), et::f16(mat_k->get()), et::f16(mat_v->cols->get()),
                              model->kdim, model->kdim, mat_v->ldm, mat_v->col_id->get(),
                              mat_v->head_ptr->get(), mat_v->nnz_col, et::f16(mat_z->get()), model->vdim,
                              et::f16(run.mask), run.lens, run.batch, model->seq_len, model->nhead, hd,
                              model->vdim / model->nhead, scale, run.causal ? ET_MHA_CAUSAL : 0, run.stream));
}

// Attention followed by the tile-sparse output projection
// (Attention/kernel_fuseO.h:6-9, Attention/kernel_fuseO.cu:254-290).  The
// reference joins the two with a grid-wide barrier inside one cooperative
// launch; here they are two back-to-back launches on one stream, which is the
// faster form on this device (8 against 25 us for one sequence of 128 tokens),
// or, with run.one_launch, the one launch of et_mha_fuseo_f16.
inline void Multihead_atttion_fuseO(half *mat_q, half *mat_k, half *mat_v, const half *mask, half *mat_z,
                                    const int *row_ptr, const int *row_offset, const half *data,
                                    const half *bias, std::shared_ptr<Model_t> model, half *out,
                                    et::AttnRun run = et::AttnRun()) {
    if (mask && !run.mask) run.mask = mask;
    if (run.one_launch) {
        const int hd = model->kdim / model->nhead;
        et::require(model->vdim == model->kdim, "fused attention: vdim must equal kdim");
        const float scale = run.scale != 0.0f ? run.scale : 1.0f / std::sqrt((float)hd);
        etChk(et_mha_fuseo_f16(et::f16(mat_q), et::f16(mat_k), et::f16(mat_v), model->kdim, model->kdim, model->vdim,
                               et::f16(mat_z), model->vdim, et::f16(run.mask), run.lens, run.batch, model->seq_len,
                               model->nhead, hd, scale, run.causal ? ET_MHA_CAUSAL : 0, row_ptr, row_offset, et::f16(data),
                               et::f16(bias), et::f16(out), model->emdim, run.stream));
        return;
    }
    et::fused_mha(mat_q, mat_k, mat_v, model->kdim, model->kdim, model->vdim, mat_z, model->vdim, *model, run);
    etChk(et_linear_bsr16_f16(row_ptr, row_offset, et::f16(data), et::f16(bias), et::f16(mat_z), et::f16(out),
                              run.batch * model->seq_len, model->vdim, model->emdim, ET_ACT_NONE, run.stream));
}

template <typename T> struct __matv_helper { using type = ptr_t; };
template <> struct __matv_helper<Prune_attn> { using type = col_mat; };

namespace et {

// A binary32 sum (projection + bias + residual) that still has to be normalised, as one layer hands
// it to the next in the split-normalisation form: the sum, its row sums per block-row group, and
// the SkipLayerNorm parameters to apply.
struct SplitSum {
    const float *v = nullptr;
    const float *stats = nullptr;
    int groups = 0;
    const half *gamma = nullptr, *beta = nullptr;
    float eps = 1e-5f;
};

// Mask / padding state shared by both Attention forms and FusedAttention.
class AttnState {
  public:
    AttnState(std::shared_ptr<Model_t> m, int batch) : model_(std::move(m)), batch_(batch) {
        require(batch >= 1, "Attention: batch must be at least 1");
        require(model_->nhead > 0 && model_->kdim % model_->nhead == 0, "Attention: kdim % nhead != 0");
    }
    // additive [S x S] mask from host memory (the reference's layout); nullptr removes it
    void set_mask(const half *host_mask) {
        if (!host_mask) { mask_.reset(); return; }
        const std::size_t n = (std::size_t)model_->seq_len * model_->seq_len;
        mask_ = std::make_unique<ptr_t>(host_mask, n);
    }
    void set_causal(bool on) { causal_ = on; }
    // right padding: keys >= lens[b] of sequence b are ignored; nullptr removes it
    void set_lens(const int *host_lens) {
        if (!host_lens) { lens_.reset(); return; }
        lens_ = std::make_unique<DeviceBuffer<int>>(host_lens, (std::size_t)batch_);
    }
    int batch() const { return batch_; }
    int rows() const { return batch_ * model_->seq_len; }
    AttnRun run(stream_t stream) const {
        AttnRun r;
        r.batch = batch_;
        r.lens = lens_ ? lens_->get() : nullptr;
        r.mask = mask_ ? mask_->get() : nullptr;
        r.causal = causal_;
        r.stream = stream;
        return r;
    }

  protected:
    std::shared_ptr<Model_t> model_;
    int batch_;
    bool causal_ = false;
    std::unique_ptr<ptr_t> mask_;
    std::unique_ptr<DeviceBuffer<int>> lens_;
};

}  // namespace et

template <typename _config, typename = void> class Attention {};

// separate Q, K, V projections — Attention/Attention.h:57-142
template <typename _config>
class Attention<_config, std::enable_if_t<!_config::isSingleKernel>> : public et::AttnState {
    using config = _config;
    using linearQ_t = Linear<typename config::WQ_t>;
    using linearK_t = Linear<typename config::WK_t>;
    using linearV_t = Linear<typename config::WV_t>;
    using linearO_t = Linear<typename config::WO_t>;
    using mat_v_t = typename __matv_helper<typename config::attn_t>::type;
    static constexpr bool kPruned = std::is_same<typename config::attn_t, Prune_attn>::value;

    std::unique_ptr<linearQ_t> linearQ;
    std::unique_ptr<linearK_t> linearK;
    std::unique_ptr<linearV_t> linearV;
    std::unique_ptr<linearO_t> linearO;
    std::unique_ptr<ptr_t> mat_k, mat_q, mat_qk, mat_z;
    std::unique_ptr<mat_v_t> mat_v;
    std::shared_ptr<Model_t> model;

  public:
    Attention(std::unique_ptr<linearQ_t> _linearQ, std::unique_ptr<linearK_t> _linearK,
              std::unique_ptr<linearV_t> _linearV, std::unique_ptr<linearO_t> _linearO,
              std::shared_ptr<Model_t> _model, int batch = 1)
        : et::AttnState(_model, batch), linearQ(std::move(_linearQ)), linearK(std::move(_linearK)),
          linearV(std::move(_linearV)), linearO(std::move(_linearO)), model(_model) {
        static_assert(std::is_same<typename config::W_t, void>::value, "separate-QKV form");
        const std::size_t T = (std::size_t)rows();
        mat_k = std::make_unique<ptr_t>(T * model->kdim);
        mat_q = std::make_unique<ptr_t>(T * model->kdim);
        mat_z = std::make_unique<ptr_t>(T * model->vdim);
        if constexpr (std::is_same<typename config::attn_t, Norm_attn>::value)
            mat_qk = std::make_unique<ptr_t>(T * model->seq_len * model->nhead);
        if constexpr (kPruned) {
            static_assert(std::is_same<typename config::WV_t, row_mat>::value,
                          "Prune_attn needs a row-pruned V projection");
            const int nnz = linearV->weight.nnz_row();
            mat_v = std::make_unique<col_mat>((int)T, model->vdim, nnz);
            mat_v->set_metadata(*linearV->weight.row_id, nnz, model->nhead, model->vdim);
        } else {
            mat_v = std::make_unique<ptr_t>(T * model->vdim);
        }
    }

    void forward(half *out, half *query, half *key, half *value, et::stream_t stream = nullptr) {
        linearQ->forward(mat_q->get(), query, stream);
        linearK->forward(mat_k->get(), key, stream);
        linearV->forward(mat_v->get(), value, stream);
        const et::AttnRun r = run(stream);
        if constexpr (std::is_same<OTF_attn_Ofused, typename config::attn_t>::value) {
            static_assert(std::is_same<typename config::WO_t, tile_mat>::value,
                          "the O-fused form needs a tile-sparse output projection");
            // what Multihead_atttion_fuseO does, with the projection through the Linear object (which
            // may hold a plan or a dense image of its weight)
            et::fused_mha(mat_q->get(), mat_k->get(), mat_v->get(), model->kdim, model->kdim, model->vdim,
                          mat_z->get(), model->vdim, *model, r);
            linearO->forward(out, mat_z->get(), stream);
        } else {
            Multihead_atttion<typename config::attn_t>(mat_q.get(), mat_k.get(), mat_v.get(), mat_qk.get(),
                                                       nullptr, mat_z.get(), model, r);
            linearO->forward(out, mat_z->get(), stream);
        }
    }

    // the same with the output projection stored as binary32 (mixed-precision layer);
    // scratch16 [rows x emdim] is used when linearO's container has no binary32 store
    void forward_f32(float *out, half *query, half *key, half *value, half *scratch16,
                     et::stream_t stream = nullptr) {
        static_assert(!std::is_same<OTF_attn_Ofused, typename config::attn_t>::value,
                      "the O-fused form has no binary32 output");
        linearQ->forward(mat_q->get(), query, stream);
        linearK->forward(mat_k->get(), key, stream);
        linearV->forward(mat_v->get(), value, stream);
        Multihead_atttion<typename config::attn_t>(mat_q.get(), mat_k.get(), mat_v.get(), mat_qk.get(), nullptr,
                                                   mat_z.get(), model, run(stream));
        et::linear_forward_f32(*linearO, out, mat_z->get(), scratch16, stream);
    }
};

// one projection H -> (2*kdim + vdim), attention over column slices of its output
// — Attention/Attention.h:204-266, kernel Attention/Attention_single.cu:10-108
template <typename _config>
class Attention<_config, std::enable_if_t<_config::isSingleKernel>> : public et::AttnState {
    using config = _config;
    using linearQKV_t = Linear<typename config::W_t>;
    using linearO_t = Linear<typename config::WO_t>;

    std::unique_ptr<linearQKV_t> linearQKV;
    std::unique_ptr<linearO_t> linearO;
    std::unique_ptr<ptr_t> mat_qkv, mat_z;
    std::shared_ptr<Model_t> model;
    bool fused_qkv_ = false;

  public:
    Attention(std::unique_ptr<linearQKV_t> _linearQKV, std::unique_ptr<linearO_t> _linearO,
              std::shared_ptr<Model_t> _model, int batch = 1)
        : et::AttnState(_model, batch), linearQKV(std::move(_linearQKV)), linearO(std::move(_linearO)),
          model(_model) {
        static_assert(!std::is_same<typename config::W_t, void>::value, "single-projection form");
        const std::size_t T = (std::size_t)rows();
        mat_qkv = std::make_unique<ptr_t>(T * (model->kdim * 2 + model->vdim));
        mat_z = std::make_unique<ptr_t>(T * model->vdim);
    }

    void forward(half *out, half *query, half *key, half *value, et::stream_t stream = nullptr) {
        et::require(query == key && key == value, "single-projection attention is self-attention");
        linearQKV->forward(mat_qkv->get(), query, stream);
        const int ldm = model->kdim * 2 + model->vdim;
        half *Q = mat_qkv->get();
        half *K = Q + model->kdim;
        half *V = K + model->kdim;
        et::fused_mha(Q, K, V, ldm, ldm, ldm, mat_z->get(), model->vdim, *model, run(stream));
        linearO->forward(out, mat_z->get(), stream);
    }

    // Split normalisation (mixed-precision layer, tile-sparse projections): the QKV projection
    // normalises the un-normalised result of the previous layer (`in`, or takes x16 when there is
    // none), the output projection adds the residual — that normalisation again, formed in its
    // epilogue, or x32 — and leaves the binary32 sum v1 with its row sums.
    bool split_ok() const {
        if constexpr (std::is_same<linearQKV_t, Linear<tile_mat>>::value && std::is_same<linearO_t, Linear<tile_mat>>::value)
            return linearQKV->split_consumer_ok() && linearO->split_producer_ok();
        else
            return false;
    }
    void prepare_split(int nwave = 0) {
        if constexpr (std::is_same<linearQKV_t, Linear<tile_mat>>::value && std::is_same<linearO_t, Linear<tile_mat>>::value) {
            linearQKV->prepare_split_consumer(nwave);
            linearO->prepare_split_producer(nwave);
        }
    }
    // The QKV projection inside the attention kernel (one launch instead of two) for the layers whose input is
    // a previous layer's un-normalised sum: sequences up to 128 tokens, heads of 64, a 768-wide model.
    // true when forward_split() will run that way.
    // gamma, beta: the affine vectors of the normalisation whose result this attention will be given (the
    // previous layer's second SkipLayerNorm), folded into the pack where they are known; forward_split() must then
    // be given exactly these.
    bool prepare_fused_qkv(const half *gamma = nullptr, const half *beta = nullptr) {
        if constexpr (std::is_same<linearQKV_t, Linear<tile_mat>>::value) {
            const int hd = model->kdim / model->nhead;
            if (model->vdim != model->kdim ||
                et_norm_qkv_mha_f32in_supported(batch(), model->seq_len, (int)linearQKV->in_size, model->nhead, hd) != 1)
                return false;
            fused_qkv_ = linearQKV->prepare_qkv_heads(model->nhead, gamma, beta);
            return fused_qkv_;
        } else {
            return false;
        }
    }
    bool fused_qkv() const { return fused_qkv_; }
    // The pieces a caller needs to run this attention as part of a chain launch (et_encoder_chain_f32):
    // the two projections, the buffers between them, and the attention kernel on its own.
    linearQKV_t &qkv_linear() { return *linearQKV; }
    linearO_t &o_linear() { return *linearO; }
    half *qkv_buffer() { return mat_qkv->get(); }
    half *z_buffer() { return mat_z->get(); }
    void core(et::stream_t stream = nullptr) {
        const int ldm = model->kdim * 2 + model->vdim;
        half *Q = mat_qkv->get();
        half *K = Q + model->kdim;
        half *V = K + model->kdim;
        et::fused_mha(Q, K, V, ldm, ldm, ldm, mat_z->get(), model->vdim, *model, run(stream));
    }
    void forward_split(float *v1, float *stats1, int *groups1, float *fin_in, const et::SplitSum *in, const float *x32,
                       half *x16, et::stream_t stream = nullptr) {
        if constexpr (std::is_same<linearQKV_t, Linear<tile_mat>>::value && std::is_same<linearO_t, Linear<tile_mat>>::value) {
            if (in && fused_qkv_) {
                const et::AttnRun r = run(stream);
                const float scale = r.scale != 0.0f ? r.scale : 1.0f / std::sqrt((float)(model->kdim / model->nhead));
                linearQKV->forward_norm_qkv_mha(mat_z->get(), model->vdim, in->v, in->stats, in->groups, in->gamma, in->beta,
                                                in->eps, fin_in, r.mask, r.lens, r.batch, model->seq_len, scale,
                                                r.causal ? ET_MHA_CAUSAL : 0, stream);
            } else {
                if (in)
                    linearQKV->forward_norm_f32in(mat_qkv->get(), in->v, in->stats, in->groups, in->gamma, in->beta,
                                                  in->eps, fin_in, nullptr, nullptr, ET_ACT_NONE, stream);
                else
                    linearQKV->forward(mat_qkv->get(), x16, stream);
                const int ldm = model->kdim * 2 + model->vdim;
                half *Q = mat_qkv->get();
                half *K = Q + model->kdim;
                half *V = K + model->kdim;
                et::fused_mha(Q, K, V, ldm, ldm, ldm, mat_z->get(), model->vdim, *model, run(stream));
            }
            if (!in && !x32)  // first layer, residual = the binary16 input itself
                linearO->forward_resid16_stats_f32(v1, stats1, groups1, mat_z->get(), x16, stream);
            else
                linearO->forward_resid_stats_f32(v1, stats1, groups1, mat_z->get(), in ? in->v : x32,
                                                 in ? fin_in : nullptr, in ? in->gamma : nullptr, in ? in->beta : nullptr,
                                                 stream);
        } else {
            (void)v1; (void)stats1; (void)groups1; (void)fin_in; (void)in; (void)x32; (void)x16; (void)stream;
            et::require(false, "Attention: the split normalisation needs tile-sparse projections");
        }
    }

    // the same with the output projection stored as binary32 (mixed-precision layer)
    void forward_f32(float *out, half *query, half *key, half *value, half *scratch16,
                     et::stream_t stream = nullptr) {
        et::require(query == key && key == value, "single-projection attention is self-attention");
        linearQKV->forward(mat_qkv->get(), query, stream);
        const int ldm = model->kdim * 2 + model->vdim;
        half *Q = mat_qkv->get();
        half *K = Q + model->kdim;
        half *V = K + model->kdim;
        et::fused_mha(Q, K, V, ldm, ldm, ldm, mat_z->get(), model->vdim, *model, run(stream));
        et::linear_forward_f32(*linearO, out, mat_z->get(), scratch16, stream);
    }
};
