// Encoder-stack handle behind the C ABI (et_model_*): assembles the C++ class
// layer (Linear / Attention / SkipLayerNorm / Encoder, include/et/*.h) from host
// weights the way the reference's example does (example/main.cu:24-182), chains
// the layers (example/main.cu:175-177) and replays the whole stack as one HIP
// graph.
#include <array>
#include <memory>
#include <string>
#include <vector>

#include "et/Encoder.h"
#include "et/weights.hpp"

namespace {

using et::stream_t;

struct ILayer {
    virtual ~ILayer() = default;
    virtual void forward(half *out, half *src, stream_t stream) = 0;
    virtual void enable_mixed() = 0;
    virtual void forward_mixed(float *out32, half *out16, const float *src32, half *src16, stream_t stream) = 0;
    virtual bool split_ok() const = 0;
    virtual void enable_split() = 0;
    virtual bool enable_fused_qkv(const half *gamma, const half *beta) = 0;
    virtual const half *norm2_gamma() const = 0;
    virtual const half *norm2_beta() const = 0;
    virtual et::SplitSum forward_split(const et::SplitSum *in, const float *x32, half *x16, stream_t stream) = 0;
    virtual void finish_split(float *out32, half *out16, const et::SplitSum &s, stream_t stream) = 0;
    virtual bool chain_parts(et::ChainParts &p) = 0;
    virtual void chain_qkv_first(half *x16, stream_t stream) = 0;
    virtual void chain_attention(stream_t stream) = 0;
    virtual et::AttnState &attn() = 0;
};

template <typename EncoderT> struct LayerOf final : ILayer {
    std::unique_ptr<EncoderT> enc;
    explicit LayerOf(std::unique_ptr<EncoderT> e) : enc(std::move(e)) {}
    void forward(half *out, half *src, stream_t stream) override { enc->forward_f16(out, src, stream); }
    void enable_mixed() override { enc->enable_mixed(); }
    void forward_mixed(float *out32, half *out16, const float *src32, half *src16, stream_t stream) override {
        enc->forward_mixed(out32, out16, src32, src16, stream);
    }
    bool split_ok() const override { return enc->split_ok(); }
    void enable_split() override { enc->enable_split(); }
    bool enable_fused_qkv(const half *gamma, const half *beta) override { return enc->enable_fused_qkv(gamma, beta); }
    const half *norm2_gamma() const override { return enc->norm2_gamma(); }
    const half *norm2_beta() const override { return enc->norm2_beta(); }
    et::SplitSum forward_split(const et::SplitSum *in, const float *x32, half *x16, stream_t stream) override {
        return enc->forward_split(in, x32, x16, stream);
    }
    void finish_split(float *out32, half *out16, const et::SplitSum &s, stream_t stream) override {
        enc->finish_split(out32, out16, s, stream);
    }
    bool chain_parts(et::ChainParts &p) override { return enc->chain_parts(p); }
    void chain_qkv_first(half *x16, stream_t stream) override { enc->chain_qkv_first(x16, stream); }
    void chain_attention(stream_t stream) override { enc->chain_attention(stream); }
    et::AttnState &attn() override { return enc->attention(); }
};

// One weight matrix as handed over by the caller (host memory).
struct HostMatrix {
    enum Kind { None, Bsr16, Dense } kind = None;
    std::vector<int> row_ptr, column;
    std::vector<half> data;  // tiles [ntile][256] or dense [out][in]
    std::vector<half> bias;
};

struct HostLayer {
    std::array<HostMatrix, 4> w;  // ET_W_QKV, ET_W_O, ET_W_FF1, ET_W_FF2
    std::array<std::vector<half>, 2> gamma, beta;
};

using tile_attn_cfg = Attention_config<tile_mat, tile_mat, tile_mat, tile_mat, OTF_attn_full, true, false>;
using dense_attn_cfg = Attention_config<base_mat, base_mat, base_mat, base_mat, OTF_attn_full, true, false>;

struct Dims {
    int out, in;
};

}  // namespace

struct et_model_s {
    et_model_desc desc{};
    std::shared_ptr<Model_t> model;
    std::vector<HostLayer> host;
    std::vector<std::unique_ptr<ILayer>> layers;
    // layer i writes ring slot i % kRing, layer i + 1 reads it; a slot is written again kRing layers on
    static constexpr int kRing = 4;
    std::unique_ptr<et::DeviceBuffer<half>> pp[kRing];
    std::unique_ptr<et::DeviceBuffer<float>> pp32[kRing];  // mixed precision: the residual stream between layers
    std::unique_ptr<et::DeviceBuffer<half>> warm;      // result of the eager pass that precedes a capture
    std::vector<int> lens;   // empty = no padding
    std::vector<half> mask;  // empty = no additive mask
    bool finalized = false;
    bool split = false;  // mixed precision with SkipLayerNorm folded into the projections
    bool fused_qkv = false;  // and the QKV projection of every layer after the first inside its attention kernel
    // split, with everything between two attention kernels in one launch (et_encoder_chain_f32):
    // one description per layer and the barrier counters of all layers, cleared at the start of a forward
    bool chain = false;
    std::vector<et_chain_desc> chain_desc;
    std::unique_ptr<et::DeviceBuffer<int>> chain_sync;

    stream_t own_stream = nullptr;
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
    ~et_model_s() {
        drop_graph();
        if (own_stream) (void)et_stream_destroy(own_stream);
    }
};

namespace {

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

template <typename MAT> std::unique_ptr<Linear<MAT>> make_linear(const HostMatrix &m, Dims d, int rows);

template <> std::unique_ptr<Linear<tile_mat>> make_linear<tile_mat>(const HostMatrix &m, Dims d, int rows) {
    tile_mat w(m.row_ptr, m.column, m.data, d.in / 16);
    et::require(w.blk_row_num == d.out / 16, "BSR weight: row_ptr length does not match the output width");
    return std::make_unique<Linear<tile_mat>>(d.in, d.out, std::move(w), m.bias.data(), rows);
}

template <> std::unique_ptr<Linear<base_mat>> make_linear<base_mat>(const HostMatrix &m, Dims d, int rows) {
    return std::make_unique<Linear<base_mat>>(d.in, d.out, base_mat(m.data), m.bias.data(), rows);
}

template <typename MAT, typename attn_cfg, typename ACT>
std::unique_ptr<ILayer> build_layer(et_model_s &m, const HostLayer &h) {
    // the layer body of Encoder<Encoder_config<attn_cfg, MAT, MAT, ACT>> without that class's own choice of
    // precision: the model's `mixed` field decides here which buffers a layer gets
    using enc_t = et::EncoderLayer<Attention<attn_cfg>, Linear<MAT>, Linear<MAT>, ACT>;
    const int rows = m.rows();
    auto lqkv = make_linear<MAT>(h.w[ET_W_QKV], m.dims(ET_W_QKV), rows);
    auto lo = make_linear<MAT>(h.w[ET_W_O], m.dims(ET_W_O), rows);
    auto attn = std::make_unique<Attention<attn_cfg>>(std::move(lqkv), std::move(lo), m.model, m.desc.batch);
    attn->set_causal(m.desc.causal != 0);
    auto ln1 = std::make_unique<SkipLayerNorm>(h.gamma[0].data(), h.beta[0].data(), m.desc.emdim, m.desc.eps);
    auto ln2 = std::make_unique<SkipLayerNorm>(h.gamma[1].data(), h.beta[1].data(), m.desc.emdim, m.desc.eps);
    auto l1 = make_linear<MAT>(h.w[ET_W_FF1], m.dims(ET_W_FF1), rows);
    auto l2 = make_linear<MAT>(h.w[ET_W_FF2], m.dims(ET_W_FF2), rows);
    auto enc = std::make_unique<enc_t>(std::move(attn), std::move(ln1), std::move(ln2), std::move(l1),
                                       std::move(l2), m.model);
    return std::make_unique<LayerOf<enc_t>>(std::move(enc));
}

template <typename MAT, typename attn_cfg> std::unique_ptr<ILayer> build_layer_act(et_model_s &m, const HostLayer &h) {
    if (m.desc.act == ET_ACT_RELU) return build_layer<MAT, attn_cfg, RELU_OP>(m, h);
    return build_layer<MAT, attn_cfg, GELU_OP>(m, h);
}

void apply_attention_state(et_model_s &m) {
    for (auto &l : m.layers) {
        l->attn().set_lens(m.lens.empty() ? nullptr : m.lens.data());
        l->attn().set_mask(m.mask.empty() ? nullptr : m.mask.data());
    }
}

void check_layer_index(const et_model_s *m, int layer) {
    et::require(m != nullptr, "et_model: NULL handle");
    et::require(layer >= 0 && layer < m->desc.nlayer, "et_model: layer index out of range");
}

// Mixed precision: the binary16 input is widened once, every layer hands the next one its result
// in both forms (binary32 residual, binary16 operand), the last one writes binary16 to `out`.
// The same with SkipLayerNorm folded into the neighbouring projections (five launches per layer):
// every layer hands the next one its un-normalised binary32 result with its row sums.
// The descriptions of the chain launches, or false when some layer has no such form.  Layer i's
// launch holds its output projection and FFN and layer i + 1's QKV projection.
bool build_chain(et_model_s &m) {
    const int n = (int)m.layers.size();
    std::vector<et::ChainParts> parts((size_t)n);
    for (int i = 0; i < n; i++)
        if (!m.layers[(size_t)i]->chain_parts(parts[(size_t)i])) return false;
    m.chain_sync = std::make_unique<et::DeviceBuffer<int>>((size_t)n * ET_CHAIN_SYNC_WORDS);
    m.chain_desc.assign((size_t)n, et_chain_desc{});
    for (int i = 0; i < n; i++) {
        const et::ChainParts &p = parts[(size_t)i];
        et_chain_desc &d = m.chain_desc[(size_t)i];
        d.o = p.o;
        d.bias_o = et::f16(p.bias_o);
        d.Z = et::f16(p.Z);
        if (i > 0) {  // the residual is LayerNorm2 of the previous layer's sum, formed from the statistics
                      // this layer's QKV projection left
            const et::ChainParts &q = parts[(size_t)i - 1];
            d.resid = q.V2;
            d.resid_fin = p.fin_in;
            d.resid_gamma = et::f16(q.gamma2);
            d.resid_beta = et::f16(q.beta2);
        }  // i == 0: resid16 = the model's input, set at run time
        d.V1 = p.V1;
        d.stats1 = p.stats1;
        d.up = p.up;
        d.bias_up = et::f16(p.bias_up);
        d.gamma1 = et::f16(p.gamma1);
        d.beta1 = et::f16(p.beta1);
        d.eps1 = p.eps1;
        d.fin1 = p.fin1;
        d.H = et::f16(p.H);
        d.act = p.act;
        d.down = p.down;
        d.bias_down = et::f16(p.bias_down);
        d.V2 = p.V2;
        d.stats2 = p.stats2;
        if (i + 1 < n) {
            const et::ChainParts &nx = parts[(size_t)i + 1];
            d.qkv = nx.qkv;
            d.bias_qkv = et::f16(nx.bias_qkv);
            d.gamma2 = et::f16(p.gamma2);
            d.beta2 = et::f16(p.beta2);
            d.eps2 = p.eps2;
            d.fin2 = nx.fin_in;
            d.QKV = et::f16(nx.QKV);
        }
        d.T = m.rows();
        d.sync = reinterpret_cast<uint32_t *>(m.chain_sync->get()) + (size_t)i * ET_CHAIN_SYNC_WORDS;
        et_chain_desc probe = d;
        if (i == 0) probe.resid16 = d.Z;  // any pointer: only the shapes are looked at
        if (et_encoder_chain_supported(&probe) != 1) return false;
    }
    return true;
}

// Two launches per layer: the attention kernel, and one chain launch for everything up to the next
// layer's QKV projection.
void run_layers_chain(et_model_s &m, half *out, half *in, stream_t stream) {
    const int n = (int)m.layers.size();
    etChk(et_fill_i32(m.chain_sync->get(), m.chain_sync->size, 0, stream));
    m.layers[0]->chain_qkv_first(in, stream);
    et::SplitSum carry;
    for (int i = 0; i < n; i++) {
        m.layers[(size_t)i]->chain_attention(stream);
        et_chain_desc d = m.chain_desc[(size_t)i];
        if (i == 0) d.resid16 = et::f16(in);
        int groups2 = 0;
        etChk(et_encoder_chain_f32(&d, &groups2, stream));
        carry.v = d.V2;
        carry.stats = d.stats2;
        carry.groups = groups2;
    }
    // the last layer's sum is normalised by its second LayerNorm
    et::ChainParts last;
    (void)m.layers[(size_t)n - 1]->chain_parts(last);
    carry.gamma = last.gamma2;
    carry.beta = last.beta2;
    carry.eps = last.eps2;
    m.layers[(size_t)n - 1]->finish_split(nullptr, out, carry, stream);
}

// true when every chain launch of the last forward ran as it must (blocking)
bool chain_ran_clean(et_model_s &m, std::string &why) {
    const int n = (int)m.layers.size();
    for (int i = 0; i < n; i++) {
        int gave_up = 0, misplaced = 0;
        etChk(et_encoder_chain_status(m.chain_desc[(size_t)i].sync, &gave_up, &misplaced));
        if (gave_up || misplaced) {
            why = "layer " + std::to_string(i) + ": " + std::to_string(gave_up) + " workgroups gave up at a barrier, " +
                  std::to_string(misplaced) + " ran on another XCD than the rest of their group";
            return false;
        }
    }
    return true;
}

void run_layers_split(et_model_s &m, half *out, half *in, stream_t stream) {
    if (m.chain) return run_layers_chain(m, out, in, stream);
    const int n = (int)m.layers.size();
    // the first layer adds the binary16 input as its residual: no widened copy
    et::SplitSum carry;
    for (int i = 0; i < n; i++)
        carry = m.layers[(size_t)i]->forward_split(i ? &carry : nullptr, nullptr, in, stream);
    m.layers[(size_t)n - 1]->finish_split(nullptr, out, carry, stream);
}

void run_layers_mixed(et_model_s &m, half *out, half *in, stream_t stream) {
    if (m.split) return run_layers_split(m, out, in, stream);
    const int n = (int)m.layers.size();
    const std::size_t elems = (std::size_t)m.rows() * m.desc.emdim;
    constexpr int R = et_model_s::kRing;
    etChk(et_f16_to_f32(m.pp32[R - 1]->get(), et::f16(in), elems, stream));
    const float *src32 = m.pp32[R - 1]->get();
    half *src16 = in;
    for (int i = 0; i < n; i++) {
        const bool last = i == n - 1;
        float *dst32 = last ? nullptr : m.pp32[i % R]->get();
        half *dst16 = last ? out : m.pp[i % R]->get();
        m.layers[(size_t)i]->forward_mixed(dst32, dst16, src32, src16, stream);
        src32 = dst32;
        src16 = dst16;
    }
}

void run_layers(et_model_s &m, half *out, half *in, stream_t stream) {
    if (m.desc.mixed) return run_layers_mixed(m, out, in, stream);
    const int n = (int)m.layers.size();
    half *src = in;
    for (int i = 0; i < n; i++) {
        half *dst = (i == n - 1) ? out : m.pp[i % et_model_s::kRing]->get();
        m.layers[(size_t)i]->forward(dst, src, stream);
        src = dst;
    }
}

std::vector<half> to_half(const float *src, size_t n) {
    std::vector<half> v(n);
    for (size_t i = 0; i < n; i++) v[i] = static_cast<half>(src[i]);
    return v;
}
std::vector<half> to_half(const et_f16 *src, size_t n) {
    std::vector<half> v(n);
    if (n) std::memcpy(v.data(), src, n * sizeof(half));  // an empty vector's data() may be null
    return v;
}

template <typename T>
int set_bsr16(et_model m, int layer, int which, const int32_t *row_ptr, const int32_t *column, const T *data,
              int ntile, const T *bias) {
    return guarded([&]() -> int {
        check_layer_index(m, layer);
        et::require(!m->finalized, "et_model: weights cannot change after et_model_finalize");
        et::require(which >= ET_W_QKV && which <= ET_W_FF2, "et_model_set_bsr16: bad matrix selector");
        et::require(row_ptr && ntile >= 0 && (ntile == 0 || (column && data)), "et_model_set_bsr16: NULL pointer");
        const Dims d = m->dims(which);
        et::require(d.out % 16 == 0 && d.in % 16 == 0, "et_model_set_bsr16: model widths must be multiples of 16");
        HostMatrix &w = m->host[(size_t)layer].w[(size_t)which];
        w.kind = HostMatrix::Bsr16;
        w.row_ptr.assign(row_ptr, row_ptr + d.out / 16 + 1);
        w.column.assign(column, column + ntile);
        w.data = to_half(data, (size_t)ntile * 256);
        w.bias = bias ? to_half(bias, (size_t)d.out) : std::vector<half>((size_t)d.out, half_zero);
        et::fmt::validate_bsr16(w.row_ptr, w.column, (size_t)ntile, d.in / 16);
        return ET_OK;
    });
}

template <typename T>
int set_dense(et_model m, int layer, int which, const T *W, const T *bias) {
    return guarded([&]() -> int {
        check_layer_index(m, layer);
        et::require(!m->finalized, "et_model: weights cannot change after et_model_finalize");
        et::require(which >= ET_W_QKV && which <= ET_W_FF2, "et_model_set_dense: bad matrix selector");
        et::require(W != nullptr, "et_model_set_dense: NULL pointer");
        const Dims d = m->dims(which);
        HostMatrix &w = m->host[(size_t)layer].w[(size_t)which];
        w.kind = HostMatrix::Dense;
        w.data = to_half(W, (size_t)d.out * d.in);
        w.bias = bias ? to_half(bias, (size_t)d.out) : std::vector<half>((size_t)d.out, half_zero);
        return ET_OK;
    });
}

template <typename T> int set_norm(et_model m, int layer, int which, const T *gamma, const T *beta) {
    return guarded([&]() -> int {
        check_layer_index(m, layer);
        et::require(!m->finalized, "et_model: weights cannot change after et_model_finalize");
        et::require((which == 0 || which == 1) && gamma && beta, "et_model_set_norm: bad arguments");
        m->host[(size_t)layer].gamma[(size_t)which] = to_half(gamma, (size_t)m->desc.emdim);
        m->host[(size_t)layer].beta[(size_t)which] = to_half(beta, (size_t)m->desc.emdim);
        return ET_OK;
    });
}

}  // namespace

extern "C" {

int et_model_create(const et_model_desc *desc, et_model *out) {
    return guarded([&]() -> int {
        et::require(desc && out, "et_model_create: NULL argument");
        *out = nullptr;
        const et_model_desc &d = *desc;
        et::require(d.kdim > 0 && d.vdim > 0 && d.seq_len > 0 && d.nhead > 0 && d.dimFF > 0 && d.emdim > 0 &&
                        d.nlayer > 0 && d.batch > 0,
                    "et_model_create: every dimension must be positive");
        et::require(d.kdim == d.vdim && d.kdim % d.nhead == 0, "et_model_create: kdim must equal vdim and divide by nhead");
        et::require(d.act == ET_ACT_RELU || d.act == ET_ACT_GELU, "et_model_create: act must be ET_ACT_RELU or ET_ACT_GELU");
        auto m = std::make_unique<et_model_s>();
        m->desc = d;
        if (m->desc.eps <= 0.0f) m->desc.eps = 1e-5f;
        m->model = std::make_shared<Model_t>(Model_t{d.kdim, d.vdim, d.seq_len, d.nhead, d.dimFF, d.emdim, d.nlayer});
        m->host.resize((size_t)d.nlayer);
        *out = m.release();
        return ET_OK;
    });
}

int et_model_set_bsr16(et_model m, int layer, int which, const int32_t *row_ptr, const int32_t *column,
                       const float *data, int ntile, const float *bias) {
    return set_bsr16<float>(m, layer, which, row_ptr, column, data, ntile, bias);
}

int et_model_set_bsr16_f16(et_model m, int layer, int which, const int32_t *row_ptr, const int32_t *column,
                           const et_f16 *data, int ntile, const et_f16 *bias) {
    return set_bsr16<et_f16>(m, layer, which, row_ptr, column, data, ntile, bias);
}

int et_model_set_dense(et_model m, int layer, int which, const float *W, const float *bias) {
    return set_dense<float>(m, layer, which, W, bias);
}

int et_model_set_dense_f16(et_model m, int layer, int which, const et_f16 *W, const et_f16 *bias) {
    return set_dense<et_f16>(m, layer, which, W, bias);
}

int et_model_set_norm(et_model m, int layer, int which, const float *gamma, const float *beta) {
    return set_norm<float>(m, layer, which, gamma, beta);
}

int et_model_set_norm_f16(et_model m, int layer, int which, const et_f16 *gamma, const et_f16 *beta) {
    return set_norm<et_f16>(m, layer, which, gamma, beta);
}

int et_model_set_lens(et_model m, const int32_t *lens_host) {
    return guarded([&]() -> int {
        et::require(m != nullptr, "et_model_set_lens: NULL handle");
        if (lens_host) m->lens.assign(lens_host, lens_host + m->desc.batch);
        else m->lens.clear();
        if (m->finalized) {
            etChk(et_device_sync());  // a replay in flight may still read the old lengths
            apply_attention_state(*m);
            m->drop_graph();          // the graph holds the old device pointers
        }
        return ET_OK;
    });
}

int et_model_set_mask(et_model m, const et_f16 *mask_host) {
    return guarded([&]() -> int {
        et::require(m != nullptr, "et_model_set_mask: NULL handle");
        const size_t n = (size_t)m->desc.seq_len * m->desc.seq_len;
        if (mask_host) m->mask = to_half(mask_host, n);
        else m->mask.clear();
        if (m->finalized) {
            etChk(et_device_sync());
            apply_attention_state(*m);
            m->drop_graph();
        }
        return ET_OK;
    });
}

int et_model_finalize(et_model m) {
    return guarded([&]() -> int {
        et::require(m != nullptr, "et_model_finalize: NULL handle");
        et::require(!m->finalized, "et_model_finalize: already finalized");
        // every device buffer of the model comes from slabs of the model's own, at fixed places in them
        struct PoolScope {
            PoolScope() { etChk(et_pool_private_begin(0)); }
            ~PoolScope() { (void)et_pool_private_end(); }
        } pool_scope;
        for (int i = 0; i < m->desc.nlayer; i++) {
            const HostLayer &h = m->host[(size_t)i];
            const HostMatrix::Kind kind = h.w[0].kind;
            for (const HostMatrix &w : h.w) {
                et::require(w.kind != HostMatrix::None, "et_model_finalize: a weight matrix was never set");
                et::require(w.kind == kind, "et_model_finalize: one layer mixes dense and BSR weights");
            }
            for (int k = 0; k < 2; k++)
                et::require(!h.gamma[(size_t)k].empty(), "et_model_finalize: a LayerNorm was never set");
            if (kind == HostMatrix::Bsr16) m->layers.push_back(build_layer_act<tile_mat, tile_attn_cfg>(*m, h));
            else m->layers.push_back(build_layer_act<base_mat, dense_attn_cfg>(*m, h));
        }
        const size_t act_elems = (size_t)m->rows() * m->desc.emdim;
        for (auto &b : m->pp) b = std::make_unique<et::DeviceBuffer<half>>(act_elems);
        m->warm = std::make_unique<et::DeviceBuffer<half>>(act_elems);
        if (m->desc.mixed) {
            for (auto &b : m->pp32) b = std::make_unique<et::DeviceBuffer<float>>(act_elems);
            for (auto &l : m->layers) l->enable_mixed();
            // mixed == 1: the engine folds SkipLayerNorm into the projections where every layer can
            m->split = (m->desc.mixed == 1 || m->desc.mixed == 3 || m->desc.mixed == 4 || m->desc.mixed == 5) && !m->layers.empty();
            for (auto &l : m->layers) m->split = m->split && l->split_ok();
            if (m->split) {
                for (auto &l : m->layers) l->enable_split();
                m->chain = m->desc.mixed == 3 && build_chain(*m);
                // The QKV projection inside the attention kernel: asked for (mixed == 4), or where it measured faster than
                // the two launches it replaces — one workgroup per (sequence, head) that reads and normalises its whole
                // sequence: 12-layer 768-wide stacks at 80 / 90 / 95 % sparsity ran 0.89 - 0.99 of the five-launch time
                // with 96 to 384 such workgroups (sequences of 32 to 128 tokens) — 96 of them on sequences of 96 or 128
                // tokens 0.99 - 1.01 —, 1.04 - 1.05 at 72 and below, 1.09 - 1.11 at 768.
                const long heads = (long)m->desc.batch * m->desc.nhead;
                const bool pays = heads >= 96 && heads <= 400;
                if ((m->desc.mixed == 4 || (m->desc.mixed == 1 && pays)) && m->layers.size() > 1) {
                    m->fused_qkv = true;
                    // (the affine part of the normalisation a layer is handed — the second one of the layer before —
                    // goes into its projection's pack)
                    for (size_t i = 1; i < m->layers.size(); i++)
                        m->fused_qkv = m->layers[i]->enable_fused_qkv(m->layers[i - 1]->norm2_gamma(), m->layers[i - 1]->norm2_beta()) &&
                                       m->fused_qkv;
                }
            }
        }
        etChk(et_stream_create(&m->own_stream));
        apply_attention_state(*m);
        m->host.clear();
        m->host.shrink_to_fit();
        m->finalized = true;
        return ET_OK;
    });
}

int et_model_forward_layer(et_model m, int layer, et_f16 *out, const et_f16 *in, et_stream stream) {
    return guarded([&]() -> int {
        check_layer_index(m, layer);
        et::require(m->finalized, "et_model_forward_layer: call et_model_finalize first");
        et::require(out && in, "et_model_forward_layer: NULL pointer");
        half *o = reinterpret_cast<half *>(out);
        half *i = reinterpret_cast<half *>(const_cast<et_f16 *>(in));
        if (m->desc.mixed) {  // one layer between binary16 buffers: the residual starts from the binary16 input
            etChk(et_f16_to_f32(m->pp32[0]->get(), in, (std::size_t)m->rows() * m->desc.emdim, stream));
            m->layers[(size_t)layer]->forward_mixed(nullptr, o, m->pp32[0]->get(), i, stream);
        } else {
            m->layers[(size_t)layer]->forward(o, i, stream);
        }
        return ET_OK;
    });
}

int et_model_forward(et_model m, et_f16 *out, const et_f16 *in, et_stream stream) {
    return guarded([&]() -> int {
        et::require(m != nullptr && m->finalized, "et_model_forward: call et_model_finalize first");
        et::require(out && in, "et_model_forward: NULL pointer");
        half *o = reinterpret_cast<half *>(out);
        half *i = reinterpret_cast<half *>(const_cast<et_f16 *>(in));
        stream_t s = stream ? stream : m->own_stream;
        if (!m->desc.use_graph) {
            run_layers(*m, o, i, s);
            return ET_OK;
        }
        if (!m->graph || m->graph_in != in || m->graph_out != out) {
            // (Re)capture for this pair of buffers.  An eager pass first runs every kernel once
            // outside capture (lazy one-time kernel setup); its result goes to a buffer of the
            // model's own, so that a caller who normalises in place (out == in) still has the
            // untouched input when the graph runs.
            m->drop_graph();
            run_layers(*m, m->warm->get(), i, s);
            etChk(et_stream_sync(s));
            std::string why;
            if (m->chain && !chain_ran_clean(*m, why)) {
                // a workgroup gave up at a barrier or ran on another XCD than its id says: separate
                // launches from here on (the eager pass is repeated so that its result is valid too)
                m->chain = false;
                et_set_last_error(("et_model_forward: the one-launch chain did not run as it must (" + why +
                                   "); using separate launches").c_str());
                run_layers(*m, m->warm->get(), i, s);
                etChk(et_stream_sync(s));
            }
            etChk(et_graph_begin_capture(s));
            try {
                run_layers(*m, o, i, s);
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

int et_model_sync(et_model m) {
    return guarded([&]() -> int {
        et::require(m != nullptr, "et_model_sync: NULL handle");
        if (m->own_stream) etChk(et_stream_sync(m->own_stream));
        return ET_OK;
    });
}

int et_model_launches_per_layer(et_model m, int *launches) {
    return guarded([&]() -> int {
        et::require(m != nullptr && launches != nullptr, "et_model_launches_per_layer: NULL argument");
        *launches = !m->finalized ? 0 : m->chain ? 2 : m->fused_qkv ? 4 : m->split ? 5 : 7;
        return ET_OK;
    });
}

int et_model_load(const char *weights_txt, const char *dir, const et_model_desc *desc, et_model *out) {
    return guarded([&]() -> int {
        et::require(weights_txt && dir && desc && out, "et_model_load: NULL argument");
        int s = et_model_create(desc, out);
        if (s != ET_OK) return s;
        std::unique_ptr<et_model_s> guard(*out);
        *out = nullptr;
        Weights weights(weights_txt, dir);
        // archive names of the exporter (example/npy2pt.py:141-174, example/main.cu:46-90)
        static const char *const mats[4] = {"self_attn.in_proj_.npz", "self_attn.out_proj..npz", "linear1..npz",
                                            "linear2..npz"};
        static const char *const norms[2] = {"norm1..npz", "norm2..npz"};
        for (int l = 0; l < desc->nlayer; l++) {
            const std::string prefix = "transformer_encoder.layers." + std::to_string(l) + ".";
            for (int w = 0; w < 4; w++) {
                const std::string f = prefix + mats[w];
                auto row_ptr = weights.load_mat<int>("row_ptr", f);
                auto column = weights.load_mat<int>("column", f);
                auto data = weights.load_mat<float>("data", f);
                auto bias = weights.load_mat<float>("B", f);
                const Dims d = guard->dims(w);
                et::require((int)row_ptr.size() == d.out / 16 + 1 && (int)bias.size() == d.out &&
                                data.size() == column.size() * 256,
                            "et_model_load: an archive does not match the model dimensions");
                etChk(et_model_set_bsr16(guard.get(), l, w, row_ptr.data(), column.data(), data.data(),
                                         (int)column.size(), bias.data()));
            }
            for (int k = 0; k < 2; k++) {
                const std::string f = prefix + norms[k];
                auto g = weights.load_mat<float>("W", f);
                auto b = weights.load_mat<float>("B", f);
                et::require((int)g.size() == desc->emdim && (int)b.size() == desc->emdim,
                            "et_model_load: a LayerNorm archive does not match emdim");
                etChk(et_model_set_norm(guard.get(), l, k, g.data(), b.data()));
            }
        }
        etChk(et_model_finalize(guard.get()));
        *out = guard.release();
        return ET_OK;
    });
}

int et_model_destroy(et_model m) {
    return guarded([&]() -> int {
        if (m) {
            (void)et_device_sync();
            delete m;
        }
        return ET_OK;
    });
}

}  // extern "C"
