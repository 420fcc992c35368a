// Transformer encoder layer (post-LN with skip connections) — the reference's
// Encoder<cfg> and Encoder_fuse<cfg> (Encoder/Encoder.h:10-139):
//   a  = attn(src)              y1  = SkipLN1(a, src)
//   f  = act(linear1(y1))       out = SkipLN2(linear2(f), y1)
// The activation is applied inside linear1's kernel epilogue (on the fp32
// accumulator) rather than as a separate pass over [rows x dimFF]; act<>() is
// still provided for callers that use it stand-alone.  forward() issues six to
// eight launches on one stream, never blocks the host and writes nothing to stdout.
//
// Precision of forward(half *out, half *src), the reference's signature: binary16 where the
// layer meets its caller and where a value is a matrix-core operand, binary32 for the residual
// stream inside the layer (both sublayer sums and both normalisations).  Twelve BERT-base layers
// called one after the other stay within 1e-2 of the binary32 mathematics that way (one binary16
// rounding per layer boundary, of values up to 8); with the residual stream rounded to binary16
// after every sublayer, as the reference stores it, they drift to 2e-2 .. 5e-2.  forward_f16() is that all-binary16 form; the environment variable
// ET_F16_RESIDUAL=1 makes forward() run it.
#pragma once
#include <cstdlib>
#include <memory>
#include <type_traits>
#include <utility>

#include "Attention.h"
#include "Fused_attention.h"
#include "LayerNorm.h"
#include "Linear.h"
#include "Model.h"
#include "SkipLayerNorm.h"

template <typename _attn, typename _l1, typename _l2, typename _act_t> struct Encoder_config {
    using attn_config = _attn;
    using linear1_config = _l1;
    using linear2_config = _l2;
    using act_t = _act_t;
};

struct RELU_OP {};
struct GELU_OP {};

namespace GELU {
// tanh-form GELU over n values (Encoder/Encoder.cu:41-68)
inline void computeGelu(et::stream_t stream, int n, const half *input, half *output) {
    etChk(et_gelu_f16(reinterpret_cast<et_f16 *>(output), reinterpret_cast<const et_f16 *>(input),
                      (std::size_t)n, stream));
}
}  // namespace GELU

namespace et {
template <typename ACT_OP_t> constexpr int act_code() {
    return std::is_same<ACT_OP_t, RELU_OP>::value ? ET_ACT_RELU
           : std::is_same<ACT_OP_t, GELU_OP>::value ? ET_ACT_GELU
                                                    : ET_ACT_NONE;
}
}  // namespace et

// in-place activation (Encoder/Encoder.h:27-37)
template <typename ACT_OP_t> void act(half *data, int size, et::stream_t stream = nullptr) {
    if constexpr (std::is_same<ACT_OP_t, RELU_OP>::value) {
        etChk(et_relu_f16(reinterpret_cast<et_f16 *>(data), reinterpret_cast<const et_f16 *>(data),
                          (std::size_t)size, stream));
    } else if constexpr (std::is_same<ACT_OP_t, GELU_OP>::value) {
        GELU::computeGelu(stream, size, data, data);
    }
}

namespace et {

// One layer's operands of a chain launch (et_chain_desc takes the projections of this layer and
// the QKV projection of the next).
struct ChainParts {
    et_bsr_pack qkv = nullptr, o = nullptr, up = nullptr, down = nullptr;
    const half *bias_qkv = nullptr, *bias_o = nullptr, *bias_up = nullptr, *bias_down = nullptr;
    half *QKV = nullptr, *Z = nullptr, *H = nullptr;
    float *fin_in = nullptr, *V1 = nullptr, *stats1 = nullptr, *fin1 = nullptr, *V2 = nullptr, *stats2 = nullptr;
    const half *gamma1 = nullptr, *beta1 = nullptr, *gamma2 = nullptr, *beta2 = nullptr;
    float eps1 = 1e-5f, eps2 = 1e-5f;
    int act = ET_ACT_NONE;
};

// The layer body shared by Encoder and Encoder_fuse.
template <typename attn_t, typename linear1_t, typename linear2_t, typename ACT_OP_t> class EncoderLayer {
  protected:
    std::unique_ptr<attn_t> attn;
    std::unique_ptr<SkipLayerNorm> LN1, LN2;
    std::unique_ptr<linear1_t> linear1;
    std::unique_ptr<linear2_t> linear2;
    std::shared_ptr<Model_t> model;
    int rows;

  public:
    DeviceBuffer<half> temp_linear;  // [rows x dimFF]
    DeviceBuffer<half> temp_attn;    // [rows x emdim]
    DeviceBuffer<half> temp_LN;      // [rows x emdim]
    // linear2's result has a buffer of its own (and so has its binary32 twin): written into
    // temp_attn, which the layer has just read, the same launch takes 1.5-2 us longer
    DeviceBuffer<half> temp_ffn;     // [rows x emdim]
    // binary32 twins of temp_attn and temp_LN, present after enable_mixed()
    std::unique_ptr<DeviceBuffer<float>> temp_attn32, temp_LN32, temp_ffn32;

    EncoderLayer(std::unique_ptr<attn_t> _attn, std::unique_ptr<SkipLayerNorm> _LN1,
                 std::unique_ptr<SkipLayerNorm> _LN2, std::unique_ptr<linear1_t> _linear1,
                 std::unique_ptr<linear2_t> _linear2, std::shared_ptr<Model_t> _model)
        : attn(std::move(_attn)), LN1(std::move(_LN1)), LN2(std::move(_LN2)), linear1(std::move(_linear1)),
          linear2(std::move(_linear2)), model(std::move(_model)), rows(attn->rows()),
          temp_linear((std::size_t)rows * model->dimFF), temp_attn((std::size_t)rows * model->emdim),
          temp_LN((std::size_t)rows * model->emdim), temp_ffn((std::size_t)rows * model->emdim) {
        require(linear1->size == rows && linear2->size == rows,
                "Encoder: the Linear layers must be built for batch * seq_len rows");
    }

    static constexpr int kFusedLnMaxRows = 256;

    attn_t &attention() { return *attn; }
    int token_rows() const { return rows; }

    // The reference's entry (Encoder/Encoder.h:81-96).  With the binary32 buffers in place
    // (prepare_wide_residual(), which the Encoder and Encoder_fuse constructors call) the residual
    // stream stays binary32 between src and out; without them this is forward_f16().
    void forward(half *out, half *src, stream_t stream = nullptr) {
        if (!wide) return forward_f16(out, src, stream);
        if (wide_split) {  // five launches and the closing normalisation
            const SplitSum s = forward_split(nullptr, nullptr, src, stream);
            return finish_split(nullptr, out, s, stream);
        }
        etChk(et_f16_to_f32(src32->get(), f16(src), (std::size_t)rows * model->emdim, stream));
        forward_mixed(nullptr, out, src32->get(), src, stream);
    }
    // Allocates what forward() needs to keep the residual stream binary32.  Not to be called while a
    // stream is being captured (it allocates, and tile-sparse layers build their packs).
    void prepare_wide_residual() {
        if (wide) return;
        if (split_ok()) {
            enable_split();
            wide_split = true;
        } else {
            enable_mixed();
            src32 = std::make_unique<DeviceBuffer<float>>((std::size_t)rows * model->emdim);
        }
        wide = true;
    }
    bool wide_residual() const { return wide; }

    // Every activation stored as binary16, the reference's own arithmetic.
    void forward_f16(half *out, half *src, stream_t stream = nullptr) {
        attn->forward(temp_attn.get(), src, src, src, stream);
        bool fused_ln1 = false;
        if constexpr (std::is_same_v<linear1_t, Linear<tile_mat>>) {
            // Up to kFusedLnMaxRows token rows SkipLayerNorm rides in the prologue of the tile-sparse
            // linear1 (one launch fewer: 12-layer forward of one sequence 376 -> 358 us); above that
            // every workgroup of a strip repeating the normalisation costs more than the launch
            // (batch 8: 544 against 534 us, batch 32: 1240 against 1184 us).
            if (rows <= kFusedLnMaxRows) {
                linear1->forward_skipln_act(temp_linear.get(), temp_LN.get(), temp_attn.get(), src, *LN1,
                                            act_code<ACT_OP_t>(), stream);
                fused_ln1 = true;
            }
        }
        if (!fused_ln1) {
            LN1->forward(temp_LN.get(), temp_attn.get(), src, rows, stream);
            linear1->forward_act(temp_linear.get(), temp_LN.get(), act_code<ACT_OP_t>(), stream);
        }
        linear2->forward(temp_ffn.get(), temp_linear.get(), stream);
        LN2->forward(out, temp_ffn.get(), temp_LN.get(), rows, stream);
    }

    // Mixed precision.  The residual stream — the layer input, both projections that feed a
    // SkipLayerNorm, and both SkipLayerNorm results — is binary32; binary16 appears only where a
    // value is a matrix-core operand (the layer input and LN1's result as Linear inputs, Q/K/V,
    // the probabilities, the attention output, the activated FFN hidden layer).  Without it the
    // rounding of the residual stream to binary16 after every sublayer is what a deep stack's
    // error consists of (12 BERT-base layers: 2e-2 against the fp32 mathematics; mixed: 1e-3).
    //   src32 / src16: the layer input in both forms;  out32 / out16: the result in both forms
    //   (either may be null).  Call enable_mixed() once before the first forward_mixed().
    void enable_mixed() {
        if (!temp_attn32) temp_attn32 = std::make_unique<DeviceBuffer<float>>((std::size_t)rows * model->emdim);
        if (!temp_LN32) temp_LN32 = std::make_unique<DeviceBuffer<float>>((std::size_t)rows * model->emdim);
        if (!temp_ffn32) temp_ffn32 = std::make_unique<DeviceBuffer<float>>((std::size_t)rows * model->emdim);
    }
    void forward_mixed(float *out32, half *out16, const float *src32, half *src16, stream_t stream = nullptr) {
        require(temp_attn32 && temp_LN32, "Encoder: call enable_mixed() before forward_mixed()");
        attn_forward_f32(temp_attn32->get(), src16, stream);
        LN1->forward_mixed(temp_LN32->get(), temp_LN.get(), temp_attn32->get(), src32, rows, stream);
        linear1->forward_act(temp_linear.get(), temp_LN.get(), act_code<ACT_OP_t>(), stream);
        linear_forward_f32(*linear2, temp_ffn32->get(), temp_linear.get(), temp_ffn.get(), stream);
        LN2->forward_mixed(out32, out16, temp_ffn32->get(), temp_LN32->get(), rows, stream);
    }

    // Split normalisation: five launches per layer, no SkipLayerNorm launch and no normalised
    // activation in memory.  The layer takes the previous layer's un-normalised result (or, first
    // layer, the input in both forms) and returns its own; finish_split() normalises the last one.
    // Same values as forward_mixed up to the rounding of the row statistics (sum and sum of squares
    // per block-row group, fp32, instead of a two-pass variance).
    bool split_ok() const {
        if constexpr (attn_has_split<attn_t>::value && std::is_same_v<linear1_t, Linear<tile_mat>> &&
                      std::is_same_v<linear2_t, Linear<tile_mat>>)
            return attn->split_ok() && linear1->split_consumer_ok() && linear2->split_producer_ok();
        else
            return false;
    }
    void enable_split() {
        enable_mixed();
        const std::size_t st = (std::size_t)16 * rows * 2;  // room for 16 block-row groups
        if (!stats1) stats1 = std::make_unique<DeviceBuffer<float>>(st);
        if (!stats2) stats2 = std::make_unique<DeviceBuffer<float>>(st);
        if (!fin_in) fin_in = std::make_unique<DeviceBuffer<float>>((std::size_t)rows * 2);
        if (!fin1) fin1 = std::make_unique<DeviceBuffer<float>>((std::size_t)rows * 2);
        if constexpr (attn_has_split<attn_t>::value && std::is_same_v<linear1_t, Linear<tile_mat>> &&
                      std::is_same_v<linear2_t, Linear<tile_mat>>) {
            // packs of 12 waves where the shape has them: what the one-launch chain takes, and as fast as
            // any other wave count in separate launches
            attn->prepare_split(kChainWaves);
            linear1->prepare_split_consumer(kChainWaves);
            linear2->prepare_split_producer(kChainWaves);
            attn->prepare_split();
            linear1->prepare_split_consumer();
            linear2->prepare_split_producer();
        }
    }
    // After enable_split(): the layer's QKV projection moves into its attention kernel (four launches per
    // layer) whenever its input is a previous layer's sum.  false where the shapes do not allow it.
    // gamma, beta: the previous layer's second normalisation (the one this layer's input carries), folded into
    // the projection where given.
    bool enable_fused_qkv(const half *gamma = nullptr, const half *beta = nullptr) {
        if constexpr (attn_has_fused_qkv<attn_t>::value) return stats1 && attn->prepare_fused_qkv(gamma, beta);
        else return false;
    }
    // the affine vectors of this layer's second normalisation, as its SplitSum hands them on
    const half *norm2_gamma() const { return LN2->gamma(); }
    const half *norm2_beta() const { return LN2->beta(); }
    static constexpr int kChainWaves = 12;
    // This layer's share of a chain launch (et_encoder_chain_f32): everything between its attention
    // kernel and the next layer's.  false when the layer's types have no such form.
    bool chain_parts(ChainParts &p) {
        if constexpr (attn_has_split<attn_t>::value && std::is_same_v<linear1_t, Linear<tile_mat>> &&
                      std::is_same_v<linear2_t, Linear<tile_mat>>) {
            auto &lq = attn->qkv_linear();
            auto &lo = attn->o_linear();
            if (!stats1 || !lq.pack_consumer || !lo.pack_producer || !linear1->pack_consumer || !linear2->pack_producer)
                return false;
            p.qkv = lq.pack_consumer.get();
            p.bias_qkv = lq.bias.get();
            p.QKV = attn->qkv_buffer();
            p.fin_in = fin_in->get();
            p.o = lo.pack_producer.get();
            p.bias_o = lo.bias.get();
            p.Z = attn->z_buffer();
            p.V1 = temp_attn32->get();
            p.stats1 = stats1->get();
            p.up = linear1->pack_consumer.get();
            p.bias_up = linear1->bias.get();
            p.gamma1 = LN1->gamma();
            p.beta1 = LN1->beta();
            p.eps1 = LN1->epsilon();
            p.fin1 = fin1->get();
            p.H = temp_linear.get();
            p.act = act_code<ACT_OP_t>();
            p.down = linear2->pack_producer.get();
            p.bias_down = linear2->bias.get();
            p.V2 = temp_ffn32->get();
            p.stats2 = stats2->get();
            p.gamma2 = LN2->gamma();
            p.beta2 = LN2->beta();
            p.eps2 = LN2->epsilon();
            return true;
        } else {
            (void)p;
            return false;
        }
    }
    // the first layer's QKV projection of the binary16 input, and the attention kernel alone
    void chain_qkv_first(half *x16, stream_t stream = nullptr) {
        if constexpr (attn_has_split<attn_t>::value) attn->qkv_linear().forward(attn->qkv_buffer(), x16, stream);
        else (void)x16, (void)stream;
    }
    void chain_attention(stream_t stream = nullptr) {
        if constexpr (attn_has_split<attn_t>::value) attn->core(stream);
        else (void)stream;
    }
    SplitSum forward_split(const SplitSum *in, const float *x32, half *x16, stream_t stream = nullptr) {
        SplitSum out;
        if constexpr (attn_has_split<attn_t>::value && std::is_same_v<linear1_t, Linear<tile_mat>> &&
                      std::is_same_v<linear2_t, Linear<tile_mat>>) {
            require(stats1 && stats2 && fin_in && fin1, "Encoder: call enable_split() before forward_split()");
            int g1 = 0, g2 = 0;
            attn->forward_split(temp_attn32->get(), stats1->get(), &g1, fin_in->get(), in, x32, x16, stream);
            linear1->forward_norm_f32in(temp_linear.get(), temp_attn32->get(), stats1->get(), g1,
                                        LN1->gamma(), LN1->beta(), LN1->epsilon(), fin1->get(), nullptr, nullptr,
                                        act_code<ACT_OP_t>(), stream);
            linear2->forward_resid_stats_f32(temp_ffn32->get(), stats2->get(), &g2, temp_linear.get(),
                                             temp_attn32->get(), fin1->get(), LN1->gamma(), LN1->beta(), stream);
            out.v = temp_ffn32->get();
            out.stats = stats2->get();
            out.groups = g2;
            out.gamma = LN2->gamma();
            out.beta = LN2->beta();
            out.eps = LN2->epsilon();
        } else {
            (void)in; (void)x32; (void)x16; (void)stream;
            require(false, "Encoder: the split normalisation needs tile-sparse projections");
        }
        return out;
    }
    void finish_split(float *out32, half *out16, const SplitSum &s, stream_t stream = nullptr) {
        etChk(et_norm_from_stats_f32in(out32, f16(out16), s.v, s.stats, s.groups, f16(s.gamma), f16(s.beta), rows,
                                       model->emdim, s.eps, stream));
    }

  protected:
    // what the drop-in classes do at the end of their constructors
    void prepare_default_precision() {
        const char *e = std::getenv("ET_F16_RESIDUAL");
        if (!(e && e[0] == '1')) prepare_wide_residual();
    }

  private:
    bool wide = false, wide_split = false;
    std::unique_ptr<DeviceBuffer<float>> src32;
    std::unique_ptr<DeviceBuffer<float>> stats1, stats2, fin_in, fin1;
    template <typename A, typename = void> struct attn_has_split : std::false_type {};
    template <typename A>
    struct attn_has_split<A, std::void_t<decltype(std::declval<A &>().forward_split(
                                 static_cast<float *>(nullptr), static_cast<float *>(nullptr), static_cast<int *>(nullptr),
                                 static_cast<float *>(nullptr), static_cast<const SplitSum *>(nullptr),
                                 static_cast<const float *>(nullptr), static_cast<half *>(nullptr),
                                 static_cast<stream_t>(nullptr)))>> : std::true_type {};
    template <typename A, typename = void> struct attn_has_fused_qkv : std::false_type {};
    template <typename A>
    struct attn_has_fused_qkv<A, std::void_t<decltype(std::declval<A &>().prepare_fused_qkv())>> : std::true_type {};
    template <typename A, typename = void> struct attn_has_f32 : std::false_type {};
    template <typename A>
    struct attn_has_f32<A, std::void_t<decltype(std::declval<A &>().forward_f32(
                               static_cast<float *>(nullptr), static_cast<half *>(nullptr),
                               static_cast<half *>(nullptr), static_cast<half *>(nullptr),
                               static_cast<half *>(nullptr), static_cast<stream_t>(nullptr)))>> : std::true_type {};
    void attn_forward_f32(float *out32, half *src16, stream_t stream) {
        if constexpr (attn_has_f32<attn_t>::value) {
            attn->forward_f32(out32, src16, src16, src16, temp_attn.get(), stream);
        } else {  // attention forms without a binary32 output projection: widen their result
            attn->forward(temp_attn.get(), src16, src16, src16, stream);
            etChk(et_f16_to_f32(out32, f16(temp_attn.get()), (std::size_t)rows * model->emdim, stream));
        }
    }
};

}  // namespace et

// Encoder/Encoder.h:49-97
template <typename _config>
class Encoder : public et::EncoderLayer<Attention<typename _config::attn_config>,
                                        Linear<typename _config::linear1_config>,
                                        Linear<typename _config::linear2_config>, typename _config::act_t> {
    using base = et::EncoderLayer<Attention<typename _config::attn_config>,
                                  Linear<typename _config::linear1_config>,
                                  Linear<typename _config::linear2_config>, typename _config::act_t>;

  public:
    template <typename... Args> explicit Encoder(Args &&...args) : base(std::forward<Args>(args)...) {
        this->prepare_default_precision();
    }
};

// Encoder with the pre-computed-VO attention (Encoder/Encoder.h:99-139): tile-sparse
// FFN, GELU.
template <typename _attn_config>
class Encoder_fuse
    : public et::EncoderLayer<FusedAttention<_attn_config>, Linear<tile_mat>, Linear<tile_mat>, GELU_OP> {
    using base = et::EncoderLayer<FusedAttention<_attn_config>, Linear<tile_mat>, Linear<tile_mat>, GELU_OP>;

  public:
    template <typename... Args> explicit Encoder_fuse(Args &&...args) : base(std::forward<Args>(args)...) {
        this->prepare_default_precision();
    }
};
