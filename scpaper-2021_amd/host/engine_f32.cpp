// Binary32 encoder-stack handle behind the C ABI (et_model_f32_*): the layer sequence of the
// reference's Encoder (Encoder/Encoder.h:81-96: attention block, SkipLayerNorm, linear1 + activation,
// linear2, SkipLayerNorm) issued through the binary32 entry points, weights dense or 16x16
// tile-sparse, chained over nlayer layers (example/main.cu:175-177) and replayed as one HIP graph.
// The reference computes in binary16 only; this is the binary32 twin of et_model_*.
#include <array>
#include <cmath>
#include <memory>
#include <vector>

#include "et/CUDA_ptr.hpp"
#include "et/format_gen.h"
#include "et/status.h"
#include "et_abi.h"

namespace {

using FBuf = et::DeviceBuffer<float>;
using IBuf = et::DeviceBuffer<int>;

struct Matrix32 {
    enum Kind { None, Bsr16, Dense } kind = None;
    std::unique_ptr<IBuf> row_ptr, column;
    std::unique_ptr<FBuf> data;  // tiles [ntile][256] or dense [out][in]
    std::unique_ptr<FBuf> bias;  // [out]
};

struct Layer32 {
    std::array<Matrix32, 4> w;  // ET_W_QKV, ET_W_O, ET_W_FF1, ET_W_FF2
    std::array<std::unique_ptr<FBuf>, 2> gamma, beta;
};

struct Dims {
    int out, in;
};

template <typename Fn> int guarded(Fn fn) {
    try {
        return fn();
    } catch (const et::Error &e) {
        et_set_last_error(e.what());
        return e.status();
    } catch (const std::exception &e) {
        et_set_last_error(e.what());
        return ET_ERR_INVALID_ARG;
    }
}

}  // namespace

struct et_model_f32_s {
    et_model_desc desc{};
    std::vector<Layer32> layers;
    std::unique_ptr<IBuf> lens;  // null = no padding
    // activations of one layer, and two buffers the layers alternate between
    std::unique_ptr<FBuf> qkv, z, attn, ln1, ff, ff2, pp[2], warm;
    bool finalized = false;
    et_stream own_stream = nullptr;
    et_graph graph = nullptr;
    const void *graph_in = nullptr;
    void *graph_out = nullptr;

    int rows() const { return desc.batch * desc.seq_len; }
    Dims dims(int which) const {
        switch (which) {
            case ET_W_QKV: return {2 * desc.kdim + desc.vdim, desc.emdim};
            case ET_W_O: return {desc.emdim, desc.vdim};
            case ET_W_FF1: return {desc.dimFF, desc.emdim};
            default: return {desc.emdim, desc.dimFF};
        }
    }
    void drop_graph() {
        if (graph) (void)et_graph_destroy(graph);
        graph = nullptr;
    }
    ~et_model_f32_s() {
        drop_graph();
        if (own_stream) (void)et_stream_destroy(own_stream);
    }
};

namespace {

void check_layer(const et_model_f32_s *m, int layer, int which, int nwhich) {
    et::require(m != nullptr, "et_model_f32: NULL handle");
    et::require(layer >= 0 && layer < m->desc.nlayer, "et_model_f32: layer index out of range");
    et::require(which >= 0 && which < nwhich, "et_model_f32: bad selector");
    et::require(!m->finalized, "et_model_f32: weights cannot change after et_model_f32_finalize");
}

void linear(const et_model_f32_s &m, const Matrix32 &w, int which, const float *x, float *y, int act, et_stream s) {
    const Dims d = m.dims(which);
    if (w.kind == Matrix32::Bsr16)
        etChk(et_linear_bsr16_f32(w.row_ptr->get(), w.column->get(), w.data->get(), w.bias->get(), x, y, m.rows(), d.in,
                                  d.out, act, s));
    else
        etChk(et_linear_dense_f32(w.data->get(), w.bias->get(), x, y, m.rows(), d.in, d.out, act, s));
}

// One layer, seven launches: QKV, attention, O, SkipLayerNorm, linear1 + activation, linear2, SkipLayerNorm.
void run_layer(et_model_f32_s &m, const Layer32 &l, float *out, const float *in, et_stream s) {
    const et_model_desc &d = m.desc;
    const int T = m.rows(), ld = 2 * d.kdim + d.vdim, hd = d.kdim / d.nhead;
    linear(m, l.w[ET_W_QKV], ET_W_QKV, in, m.qkv->get(), ET_ACT_NONE, s);
    const float *q = m.qkv->get();
    etChk(et_mha_fused_f32(q, q + d.kdim, q + 2 * d.kdim, ld, ld, ld, m.z->get(), d.vdim, nullptr,
                           m.lens ? m.lens->get() : nullptr, d.batch, d.seq_len, d.nhead, hd, 1.0f / std::sqrt((float)hd),
                           d.causal ? ET_MHA_CAUSAL : 0, s));
    linear(m, l.w[ET_W_O], ET_W_O, m.z->get(), m.attn->get(), ET_ACT_NONE, s);
    etChk(et_skip_layernorm_f32(m.ln1->get(), m.attn->get(), in, l.gamma[0]->get(), l.beta[0]->get(), T, d.emdim, d.eps, s));
    linear(m, l.w[ET_W_FF1], ET_W_FF1, m.ln1->get(), m.ff->get(), d.act, s);
    linear(m, l.w[ET_W_FF2], ET_W_FF2, m.ff->get(), m.ff2->get(), ET_ACT_NONE, s);
    etChk(et_skip_layernorm_f32(out, m.ff2->get(), m.ln1->get(), l.gamma[1]->get(), l.beta[1]->get(), T, d.emdim, d.eps, s));
}

void run_layers(et_model_f32_s &m, float *out, const float *in, et_stream s) {
    const int n = m.desc.nlayer;
    const float *src = in;
    for (int i = 0; i < n; i++) {
        float *dst = (i + 1 == n) ? out : m.pp[i & 1]->get();
        run_layer(m, m.layers[(size_t)i], dst, src, s);
        src = dst;
    }
}

}  // namespace

extern "C" {

int et_model_f32_create(const et_model_desc *desc, et_model_f32 *out) {
    return guarded([&]() -> int {
        et::require(desc && out, "et_model_f32_create: NULL pointer");
        et::require(desc->kdim > 0 && desc->vdim > 0 && desc->seq_len > 0 && desc->nhead > 0 && desc->dimFF > 0 &&
                        desc->emdim > 0 && desc->nlayer > 0 && desc->batch > 0,
                    "et_model_f32_create: sizes must be positive");
        et::require(desc->kdim == desc->vdim && desc->kdim == desc->emdim,
                    "et_model_f32_create: kdim, vdim and emdim must be equal (the layer adds its input to the projection)");
        et::require(desc->kdim % desc->nhead == 0, "et_model_f32_create: kdim must be a multiple of nhead");
        et::require(desc->act == ET_ACT_RELU || desc->act == ET_ACT_GELU, "et_model_f32_create: act must be ReLU or GELU");
        auto m = std::make_unique<et_model_f32_s>();
        m->desc = *desc;
        if (m->desc.eps <= 0.0f) m->desc.eps = 1e-5f;
        m->layers.resize((size_t)desc->nlayer);
        *out = m.release();
        return ET_OK;
    });
}

int et_model_f32_set_bsr16(et_model_f32 m, int layer, int which, const int32_t *row_ptr, const int32_t *column,
                           const float *data, int ntile, const float *bias) {
    return guarded([&]() -> int {
        check_layer(m, layer, which, 4);
        et::require(row_ptr && ntile >= 0 && (ntile == 0 || (column && data)), "et_model_f32_set_bsr16: NULL pointer");
        const Dims d = m->dims(which);
        et::require(d.out % 16 == 0 && d.in % 16 == 0, "et_model_f32_set_bsr16: model widths must be multiples of 16");
        const std::vector<int> rp(row_ptr, row_ptr + d.out / 16 + 1), col(column, column + ntile);
        et::fmt::validate_bsr16(rp, col, (size_t)ntile, d.in / 16);
        Matrix32 &w = m->layers[(size_t)layer].w[(size_t)which];
        w.kind = Matrix32::Bsr16;
        w.row_ptr = std::make_unique<IBuf>(rp);
        // an empty weight keeps one (unread) element so that every pointer handed on is valid
        w.column = ntile ? std::make_unique<IBuf>(col) : std::make_unique<IBuf>(1);
        w.data = ntile ? std::make_unique<FBuf>(data, (size_t)ntile * 256) : std::make_unique<FBuf>(256);
        w.bias = bias ? std::make_unique<FBuf>(bias, (size_t)d.out) : std::make_unique<FBuf>((size_t)d.out);
        return ET_OK;
    });
}

int et_model_f32_set_dense(et_model_f32 m, int layer, int which, const float *W, const float *bias) {
    return guarded([&]() -> int {
        check_layer(m, layer, which, 4);
        et::require(W != nullptr, "et_model_f32_set_dense: NULL pointer");
        const Dims d = m->dims(which);
        Matrix32 &w = m->layers[(size_t)layer].w[(size_t)which];
        w.kind = Matrix32::Dense;
        w.row_ptr.reset();
        w.column.reset();
        w.data = std::make_unique<FBuf>(W, (size_t)d.out * d.in);
        w.bias = bias ? std::make_unique<FBuf>(bias, (size_t)d.out) : std::make_unique<FBuf>((size_t)d.out);
        return ET_OK;
    });
}

int et_model_f32_set_norm(et_model_f32 m, int layer, int which, const float *gamma, const float *beta) {
    return guarded([&]() -> int {
        check_layer(m, layer, which, 2);
        et::require(gamma && beta, "et_model_f32_set_norm: NULL pointer");
        Layer32 &l = m->layers[(size_t)layer];
        l.gamma[(size_t)which] = std::make_unique<FBuf>(gamma, (size_t)m->desc.emdim);
        l.beta[(size_t)which] = std::make_unique<FBuf>(beta, (size_t)m->desc.emdim);
        return ET_OK;
    });
}

int et_model_f32_set_lens(et_model_f32 m, const int32_t *lens_host) {
    return guarded([&]() -> int {
        et::require(m != nullptr, "et_model_f32_set_lens: NULL handle");
        if (lens_host) {
            for (int b = 0; b < m->desc.batch; b++)
                et::require(lens_host[b] >= 0 && lens_host[b] <= m->desc.seq_len, "et_model_f32_set_lens: length out of range");
            m->lens = std::make_unique<IBuf>(lens_host, (size_t)m->desc.batch);
        } else {
            m->lens.reset();
        }
        m->drop_graph();  // a captured graph holds the old pointer
        return ET_OK;
    });
}

int et_model_f32_finalize(et_model_f32 m) {
    return guarded([&]() -> int {
        et::require(m != nullptr, "et_model_f32_finalize: NULL handle");
        et::require(!m->finalized, "et_model_f32_finalize: already finalized");
        for (const Layer32 &l : m->layers) {
            for (const Matrix32 &w : l.w) et::require(w.kind != Matrix32::None, "et_model_f32_finalize: a weight matrix was never set");
            for (int k = 0; k < 2; k++) et::require(l.gamma[(size_t)k] != nullptr, "et_model_f32_finalize: a LayerNorm was never set");
        }
        const et_model_desc &d = m->desc;
        const size_t T = (size_t)m->rows();
        m->qkv = std::make_unique<FBuf>(T * (2 * d.kdim + d.vdim));
        m->z = std::make_unique<FBuf>(T * d.vdim);
        m->attn = std::make_unique<FBuf>(T * d.emdim);
        m->ln1 = std::make_unique<FBuf>(T * d.emdim);
        m->ff = std::make_unique<FBuf>(T * d.dimFF);
        m->ff2 = std::make_unique<FBuf>(T * d.emdim);
        for (auto &b : m->pp) b = std::make_unique<FBuf>(T * d.emdim);
        m->warm = std::make_unique<FBuf>(T * d.emdim);
        etChk(et_stream_create(&m->own_stream));
        m->finalized = true;
        return ET_OK;
    });
}

int et_model_f32_forward(et_model_f32 m, float *out, const float *in, et_stream stream) {
    return guarded([&]() -> int {
        et::require(m != nullptr && m->finalized, "et_model_f32_forward: call et_model_f32_finalize first");
        et::require(out && in, "et_model_f32_forward: NULL pointer");
        et_stream s = stream ? stream : m->own_stream;
        if (!m->desc.use_graph) {
            run_layers(*m, out, in, s);
            return ET_OK;
        }
        if (!m->graph || m->graph_in != in || m->graph_out != out) {
            // (Re)capture for this pair of buffers, after an eager pass into a buffer of the model's own
            // (one-time kernel set-up happens outside the capture; out == in keeps its input).
            m->drop_graph();
            run_layers(*m, m->warm->get(), in, s);
            etChk(et_stream_sync(s));
            etChk(et_graph_begin_capture(s));
            try {
                run_layers(*m, out, in, s);
            } catch (...) {
                et_graph dead = nullptr;
                (void)et_graph_end_capture(s, &dead);
                (void)et_graph_destroy(dead);
                throw;
            }
            etChk(et_graph_end_capture(s, &m->graph));
            m->graph_in = in;
            m->graph_out = out;
        }
        etChk(et_graph_launch(m->graph, s));
        return ET_OK;
    });
}

int et_model_f32_sync(et_model_f32 m) {
    return guarded([&]() -> int {
        et::require(m != nullptr && m->finalized, "et_model_f32_sync: call et_model_f32_finalize first");
        etChk(et_stream_sync(m->own_stream));
        return ET_OK;
    });
}

int et_model_f32_destroy(et_model_f32 m) {
    if (m) {
        if (m->own_stream) (void)et_stream_sync(m->own_stream);
        delete m;
    }
    return ET_OK;
}

}  // extern "C"
