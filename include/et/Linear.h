// y = x W^T + b for every weight container — the reference's Linear<MAT>
// (Linear/Linear.h:17-167).  W is the PyTorch [out x in] matrix; x and y are
// row-major [size x features] device pointers owned by the caller; `size` (the
// number of token rows, = batch * seq_len) is fixed at construction.  Each
// forward is ONE kernel launch on the given stream: bias (and, through
// forward_act, the activation) is applied on the fp32 accumulator in the
// kernel's epilogue, and the row/column-pruned forms gather/scatter inside the
// GEMM instead of the reference's extra passes.  Nothing blocks the host.
#pragma once
#include <algorithm>
#include <cstdlib>
#include <memory>
#include <type_traits>
#include <utility>
#include <vector>

#include "CUDA_ptr.hpp"
#include "mat_type.h"

using base_mat = et::DeviceBuffer<half>;  // dense [out x in] row-major (Linear/Linear.h:9)

namespace et {
inline const et_f16 *f16(const half *p) { return reinterpret_cast<const et_f16 *>(p); }
inline et_f16 *f16(half *p) { return reinterpret_cast<et_f16 *>(p); }
}  // namespace et

template <typename MAT> class Linear;  // only the specialisations below exist

// dense weight — Linear/Linear.h:32-66
template <> class Linear<base_mat> {
  public:
    const int in_size;
    const int out_size;
    base_mat weight;
    et::DeviceBuffer<half> bias;
    int size;

    Linear(int _in_size, int _out_size, const base_mat &w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), weight(w), bias(b, (std::size_t)_out_size), size(_size) {
        et::require(w.size == (std::size_t)_in_size * _out_size, "Linear<base_mat>: weight must hold out*in values");
    }
    Linear(int _in_size, int _out_size, base_mat &&w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), weight(std::move(w)), bias(b, (std::size_t)_out_size),
          size(_size) {
        et::require(weight.size == (std::size_t)_in_size * _out_size, "Linear<base_mat>: weight must hold out*in values");
    }
    void forward(half *output, const half *input, et::stream_t stream = nullptr) const {
        forward_act(output, input, ET_ACT_NONE, stream);
    }
    void forward_act(half *output, const half *input, int act, et::stream_t stream = nullptr) const {
        etChk(et_linear_dense_f16(et::f16(weight.get()), et::f16(bias.get()), et::f16(input), et::f16(output),
                                  size, in_size, out_size, act, stream));
    }
};

namespace et {
namespace detail {
// ids (on the device) are exactly 0, 1, ..., n - 1: read back once, at construction
inline bool is_identity(const et::DeviceBuffer<int> &ids, int n) {
    if ((long long)ids.size != n) return false;
    const std::vector<int> host = ids.to_host();
    for (int i = 0; i < n; i++)
        if (host[(std::size_t)i] != i) return false;
    return true;
}
}  // namespace detail
}  // namespace et

// output-feature pruning — Linear/Linear.h:69-86, Linear/SPMM_row.cu:48-95
template <> class Linear<row_mat> {
  public:
    const uint32_t in_size;
    const uint32_t out_size;
    row_mat weight;
    et::DeviceBuffer<half> bias;
    int size;
    bool nothing_pruned = false;  // every row kept, in order: the weight is a plain dense one
    // The full-width forward of a pruned weight costs a fill of the whole result (pruned features carry their
    // bias) and a GEMM whose epilogue scatters single elements; measured at 2048 rows it beats the dense GEMM of
    // the same layer only once fewer than a tenth of the features survive.  Above that the class multiplies a
    // dense image of the weight, [out x in] with zero rows where features are pruned: the same values (a zero
    // row gives the bias alone), one launch, whole-row stores.  Built at construction; whoever rewrites
    // `weight` afterwards calls refresh().
    std::unique_ptr<et::DeviceBuffer<half>> dense_image;
    static bool wants_dense_image(long nnz_row, long out) { return nnz_row * 10 > out; }

    Linear(int _in_size, int _out_size, const row_mat &w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), weight(w), bias(b, (std::size_t)_out_size), size(_size) {
        refresh();
    }
    Linear(int _in_size, int _out_size, row_mat &&w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), weight(std::move(w)), bias(b, (std::size_t)_out_size),
          size(_size) {
        refresh();
    }
    // what the class derives from `weight`: called by the constructors, and by a caller that changed it
    // (outside any stream capture: it reads the ids back and may allocate)
    void refresh() {
        nothing_pruned = et::detail::is_identity(*weight.row_id, (int)out_size);
        dense_image.reset();
        const long nnz = weight.nnz_row();
        if (nothing_pruned || !wants_dense_image(nnz, (long)out_size)) return;
        const std::vector<int> ids = weight.row_id->to_host();
        const std::vector<half> rows = weight.rows->to_host();
        std::vector<half> image((std::size_t)out_size * in_size, static_cast<half>(0.0f));
        for (long i = 0; i < nnz; i++) {
            const long r = ids[(std::size_t)i];
            if (r < 0 || r >= (long)out_size) throw et::Error(ET_ERR_INVALID_ARG, "Linear<row_mat>: row id outside the weight");
            std::copy(rows.begin() + i * in_size, rows.begin() + (i + 1) * in_size, image.begin() + r * in_size);
        }
        dense_image = std::make_unique<et::DeviceBuffer<half>>(image);
    }
    // full-width output: pruned features carry their bias alone
    void forward(half *output, const half *input, et::stream_t stream = nullptr) const {
        forward_act(output, input, ET_ACT_NONE, stream);
    }
    void forward_act(half *output, const half *input, int act, et::stream_t stream = nullptr) const {
        if (nothing_pruned || dense_image) {  // no fill pass, no scattered stores
            const half *w = dense_image ? dense_image->get() : weight.rows->get();
            etChk(et_linear_dense_f16(et::f16(w), et::f16(bias.get()), et::f16(input),
                                      et::f16(output), size, (int)in_size, (int)out_size, act, stream));
            return;
        }
        etChk(et_linear_rowpruned_f16(et::f16(weight.rows->get()), weight.row_id->get(), weight.nnz_row(),
                                      et::f16(bias.get()), et::f16(input), et::f16(output), size,
                                      (int)in_size, (int)out_size, act, stream));
    }
    // compact output [size x nnz_row] written into a col_mat (the compact V of the
    // attention-aware path, Linear/SPMM_row.cu:78-95); the bias of each surviving
    // feature is applied (the reference leaves that line commented out).
    void forward(col_mat *output, const half *input, et::stream_t stream = nullptr) const {
        etChk(et_linear_rowpruned_compact_f16(et::f16(weight.rows->get()), weight.row_id->get(),
                                              weight.nnz_row(), et::f16(bias.get()), et::f16(input),
                                              et::f16(output->cols->get()), size, (int)in_size, stream));
    }
};

// input-feature pruning — Linear/Linear.h:115-131, Linear/SPMM_col.cu:41-69
template <> class Linear<col_mat> {
  public:
    const uint32_t in_size;
    const uint32_t out_size;
    col_mat weight;
    et::DeviceBuffer<half> bias;
    int size;
    mutable et::DeviceBuffer<half> gathered;  // [size x nnz_col] compact activations (the workspace of Linear/Linear.h:124)

    Linear(int _in_size, int _out_size, const col_mat &w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), weight(w), bias(b, (std::size_t)_out_size), size(_size),
          gathered((std::size_t)_size * weight.nnz_col) {}
    Linear(int _in_size, int _out_size, col_mat &&w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), weight(std::move(w)), bias(b, (std::size_t)_out_size),
          size(_size), gathered((std::size_t)_size * weight.nnz_col) {}
    void forward(half *output, const half *input, et::stream_t stream = nullptr) const {
        forward_act(output, input, ET_ACT_NONE, stream);
    }
    // gather the surviving input features once, then one dense GEMM with the bias and the
    // activation in its epilogue
    void forward_act(half *output, const half *input, int act, et::stream_t stream = nullptr) const {
        if (weight.nnz_col == 0 || size == 0) {
            etChk(et_linear_colpruned_f16(et::f16(weight.cols->get()), weight.col_id->get(), weight.nnz_col,
                                          et::f16(bias.get()), et::f16(input), et::f16(output), size,
                                          (int)in_size, (int)out_size, act, stream));
            return;
        }
        etChk(et_linear_colpruned_ws_f16(et::f16(weight.cols->get()), weight.col_id->get(), weight.nnz_col,
                                         et::f16(bias.get()), et::f16(input), et::f16(output),
                                         et::f16(gathered.get()), size, (int)in_size, (int)out_size, act, stream));
    }
};

// 16x16 tile pruning — Linear/Linear.h:133-151, Linear/SPMM_tile.cu:312-324
template <> class Linear<tile_mat> {
  public:
    const uint32_t in_size;
    const uint32_t out_size;
    const int size;
    tile_mat weight;
    et::DeviceBuffer<half> bias;
    // Re-ordered copy of the weight for the streaming kernel (et_bsr16_plan_create), held where
    // that kernel is the faster one: inputs too wide for an LDS-resident token strip, and wide
    // inputs at many token rows (measured: 1.6-2x at in > 5112, 1.1-1.4x at in >= 3072 from 4096 rows).
    struct PlanDeleter {
        void operator()(et_bsr_plan_s *p) const { (void)et_bsr16_plan_destroy(p); }
    };
    std::unique_ptr<et_bsr_plan_s, PlanDeleter> plan;
    static bool wants_plan(int in, int rows) { return in >= 128 && (in > 5112 || (in >= 3072 && rows >= 4096)); }
    // Copies of the weight in the order one launch of the packed kernel reads it (et_bsr16_pack_create),
    // held where that kernel applies — up to kPackMaxRows token rows, inputs that are multiples of 128
    // up to 4096: a launch whose loads are all issued at its start, with no row-pointer round trip.
    // `pack` serves forward / forward_act / forward_f32; the split normalisation of the
    // mixed-precision layer builds one more per role on prepare_split_producer / _consumer.
    struct PackDeleter {
        void operator()(et_bsr_pack_s *p) const { (void)et_bsr16_pack_destroy(p); }
    };
    using pack_ptr = std::unique_ptr<et_bsr_pack_s, PackDeleter>;
    pack_ptr pack, pack_producer, pack_consumer;
    // W_qkv ordered head by head for the attention kernel that projects Q, K and V itself
    // (et_qkv_heads_pack_create); built on prepare_qkv_heads()
    pack_ptr pack_heads;
    int heads_nhead = 0;
    const half *heads_gamma = nullptr, *heads_beta = nullptr;  // the normalisation folded into pack_heads (null: none)
    int producer_nwave = 0, consumer_nwave = 0;  // the wave counts the role packs were asked for (0: the builder's choice)
    static constexpr int kPackMaxRows = 4096;
    // Where a pack pays (measured against the unpacked kernel at 128 .. 1536 rows, 768- and 3072-wide inputs, 80 / 90 /
    // 95 % sparsity): block-rows of at least 8 tiles on average — below that a wave's fixed run of slots is mostly
    // padding (768 -> 2304 at 95 %, 128 rows: 8.6 against 3.6 us) — and either a wide input, where the unpacked
    // kernel's chain of dependent loads is long (3072 -> 768: 0.68 - 0.85 of the unpacked time at any row count), or
    // at least 256 rows (768-wide at 80 %: 1.12 - 1.37 at 128 rows, 0.89 - 1.01 from 256 on).
    bool pack_pays() const {
        return (long)weight.num_blk >= 8L * weight.blk_row_num && (in_size >= 2048 || size >= 256);
    }
    // forward / forward_act / forward_f32 take the one-strip pack up to this many rows (at 1536 rows and beyond the
    // plain call is level or 5-25 % faster)
    static constexpr int kPlainPackMaxRows = 1024;
    // From kRowLoopMinRows rows on, for inputs up to 1536 wide: the pack of the row-loop kernel (weights resident
    // in registers, token strips staged two ahead), where its launch fills the chip — at least 256 (strip, group)
    // pairs.  Measured against the plain call: 16384 x 768 -> 3072 43 against 60 us, -> 2304 32 against 45 us,
    // -> 768 16 against 20 us; 4096 x 768 -> 3072 15 against 19 us; 2048 x 768 -> 2304 7.9 against 10.5 us.
    // Serves forward / forward_act (binary16 results) and forward_f32 (binary32 results).
    pack_ptr pack_loop;
    static constexpr int kRowLoopMinRows = 2048;
    // ET_PACKED=0 in the environment keeps every Linear<tile_mat> on the unpacked kernels (for comparisons)
    static bool packed_enabled() {
        static const bool on = [] {
            const char *e = std::getenv("ET_PACKED");
            return !(e && e[0] == '0');
        }();
        return on;
    }
    // Dense image of the weight, held where the dense GEMM is the faster kernel: a matrix that
    // keeps most of its tiles (measured at 2048 rows: the tile kernel overtakes the dense one at
    // 35-50 % sparsity for 768-wide inputs, at 50 % for 3072-wide ones).  Not built when a tile
    // position occurs twice (the tile kernel adds such tiles up, an image cannot).
    std::unique_ptr<et::DeviceBuffer<half>> dense;
    std::unique_ptr<et::DeviceBuffer<half>> dense_out16;  // fp16 result ahead of the widening in forward_f32
    static bool wants_dense(int in, int out, int ntile) {
        const double kept = (double)ntile * 256.0 / ((double)in * (double)out);
        (void)in;
        return kept > 0.50;
    }

    Linear(int _in_size, int _out_size, const tile_mat &w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), size(_size), weight(w), bias(b, (std::size_t)_out_size) {
        check();
    }
    Linear(int _in_size, int _out_size, const tile_mat &w, et::DeviceBuffer<half> &b, int _size)
        : in_size(_in_size), out_size(_out_size), size(_size), weight(w), bias(b) {
        check();
    }
    Linear(int _in_size, int _out_size, tile_mat &&w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), size(_size), weight(std::move(w)),
          bias(b, (std::size_t)_out_size) {
        check();
    }
    Linear(Linear<tile_mat> &&other) = default;

    void forward(half *output, const half *const input, et::stream_t stream = nullptr) {
        forward_act(output, input, ET_ACT_NONE, stream);
    }
    void forward_act(half *output, const half *input, int act, et::stream_t stream = nullptr) {
        if (dense) {
            etChk(et_linear_dense_f16(et::f16(dense->get()), et::f16(bias.get()), et::f16(input), et::f16(output), size,
                                      (int)in_size, (int)out_size, act, stream));
            return;
        }
        if (plan) {
            etChk(et_linear_bsr16_planned_f16(plan.get(), et::f16(bias.get()), et::f16(input), et::f16(output), nullptr,
                                              size, act, stream));
            return;
        }
        if (pack_loop) {
            etChk(et_linear_bsr16_packed_f16(pack_loop.get(), et::f16(bias.get()), et::f16(input), et::f16(output), nullptr,
                                             size, act, stream));
            return;
        }
        if (pack) {
            etChk(et_linear_bsr16_packed_f16(pack.get(), et::f16(bias.get()), et::f16(input), et::f16(output), nullptr,
                                             size, act, stream));
            return;
        }
        etChk(et_linear_bsr16_f16(weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()),
                                  et::f16(bias.get()), et::f16(input), et::f16(output), size, (int)in_size,
                                  (int)out_size, act, stream));
    }
    // binary32 result (fp16 operands, fp32 accumulator stored unrounded): what the
    // mixed-precision encoder layer adds to its fp32 residual stream
    void forward_f32(float *output, const half *input, et::stream_t stream = nullptr) {
        if (dense) {  // the dense GEMM stores fp16: widened afterwards
            forward_act(dense_out16->get(), input, ET_ACT_NONE, stream);
            etChk(et_f16_to_f32(output, et::f16(dense_out16->get()), (std::size_t)size * out_size, stream));
            return;
        }
        if (plan) {
            etChk(et_linear_bsr16_planned_f16(plan.get(), et::f16(bias.get()), et::f16(input), nullptr, output, size,
                                              ET_ACT_NONE, stream));
            return;
        }
        if (pack_loop) {
            etChk(et_linear_bsr16_packed_f16(pack_loop.get(), et::f16(bias.get()), et::f16(input), nullptr, output, size,
                                             ET_ACT_NONE, stream));
            return;
        }
        if (pack) {
            etChk(et_linear_bsr16_packed_f16(pack.get(), et::f16(bias.get()), et::f16(input), nullptr, output, size,
                                             ET_ACT_NONE, stream));
            return;
        }
        etChk(et_linear_bsr16_f16_f32out(weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()),
                                         et::f16(bias.get()), et::f16(input), output, size, (int)in_size,
                                         (int)out_size, ET_ACT_NONE, stream));
    }
    // The split normalisation of the mixed-precision layer (et_linear_bsr16_resid_stats_f32 /
    // et_norm_linear_bsr16_f32in): this Linear as the producer of a binary32 sum with its row
    // sums, or as the consumer that normalises such a sum while it stages its token strip.
    bool split_producer_ok() const {
        return !dense && !plan && size > 0 && et_linear_bsr16_resid_stats_f32_supported(size, (int)in_size, (int)out_size) == 1;
    }
    bool split_consumer_ok() const {
        return !dense && !plan && size > 0 && et_norm_linear_bsr16_f32in_supported(size, (int)in_size, (int)out_size) == 1;
    }
    // Packs for the two roles (called once, outside any stream capture; a shape the packed kernel does
    // not take keeps the unpacked one)
    // (nwave: waves per workgroup the pack is built for, 0 = the builder's choice; the one-launch
    // chain of the encoder layer takes packs of 12)
    void prepare_split_producer(int nwave = 0) {
        if (!pack_producer && !dense && !plan && (pack_producer = make_pack(ET_PACK_STATS_PRODUCER, nwave)))
            producer_nwave = nwave;
    }
    void prepare_split_consumer(int nwave = 0) {
        if (!pack_consumer && !dense && !plan && (pack_consumer = make_pack(ET_PACK_NORM_CONSUMER, nwave)))
            consumer_nwave = nwave;
    }
    // This Linear as the QKV projection of `nhead` heads of 64 inside the attention kernel: false (and nothing
    // built) where that kernel does not take the weight.  Called once, outside any stream capture.
    // With gamma and beta (device pointers that stay valid, the affine vectors of the normalisation this projection
    // will be given) they are folded into the pack: W diag(gamma), bias + W beta.  A caller that rewrites them
    // calls refresh().
    bool prepare_qkv_heads(int nhead, const half *gamma = nullptr, const half *beta = nullptr) {
        if (pack_heads) return heads_nhead == nhead && heads_gamma == gamma && heads_beta == beta;
        if (dense || plan || !packed_enabled() || (long)out_size != 3L * nhead * 64) return false;
        et_bsr_pack p = nullptr;
        const int s = gamma && beta
                          ? et_qkv_heads_pack_create_folded(weight.row_ptr.get(), weight.row_offset.get(),
                                                            et::f16(weight.data.get()), et::f16(bias.get()), et::f16(gamma),
                                                            et::f16(beta), (int)in_size, nhead, &p)
                          : et_qkv_heads_pack_create(weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()),
                                                     (int)in_size, nhead, &p);
        if (s == ET_ERR_UNSUPPORTED) return false;
        etChk(s);
        pack_heads.reset(p);
        heads_nhead = nhead;
        heads_gamma = gamma && beta ? gamma : nullptr;
        heads_beta = gamma && beta ? beta : nullptr;
        return true;
    }
    // Z = attention over (Q, K, V) = normalised(V32) W^T + bias, in one launch (et_norm_qkv_mha_f32in)
    void forward_norm_qkv_mha(half *Z, int ldz, const float *V32, const float *stats, int groups, const half *gamma,
                              const half *beta, float eps, float *fin_out, const half *mask, const int *lens, int batch,
                              int seq_len, float scale, int flags, et::stream_t stream = nullptr) {
        et::require((bool)pack_heads, "Linear<tile_mat>: prepare_qkv_heads() was not called or did not apply");
        et::require(heads_gamma == nullptr || (heads_gamma == gamma && heads_beta == beta),
                    "Linear<tile_mat>: the pack was folded with another normalisation than the one it is given");
        etChk(et_norm_qkv_mha_f32in(pack_heads.get(), V32, stats, groups, et::f16(gamma), et::f16(beta), eps, fin_out,
                                    et::f16(bias.get()), et::f16(Z), ldz, et::f16(mask), lens, batch, seq_len, scale, flags,
                                    stream));
    }
    // V = input W^T + bias + residual (binary32) and stats[*groups][size][2]; the residual is
    // `resid` itself, or with resid_fin its normalisation by (resid_fin, resid_gamma, resid_beta)
    void forward_resid_stats_f32(float *V, float *stats, int *groups, const half *input, const float *resid,
                                 const float *resid_fin, const half *resid_gamma, const half *resid_beta,
                                 et::stream_t stream = nullptr) {
        if (pack_producer) {
            etChk(et_linear_bsr16_packed_resid_stats_f32(pack_producer.get(), et::f16(bias.get()), et::f16(input), resid, nullptr,
                                                         resid_fin, et::f16(resid_gamma), et::f16(resid_beta), V, stats, groups,
                                                         size, stream));
            return;
        }
        etChk(et_linear_bsr16_resid_stats_f32(weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()),
                                              et::f16(bias.get()), et::f16(input), resid, resid_fin, et::f16(resid_gamma),
                                              et::f16(resid_beta), V, stats, groups, size, (int)in_size, (int)out_size,
                                              stream));
    }
    // the same with the residual in binary16
    void forward_resid16_stats_f32(float *V, float *stats, int *groups, const half *input, const half *resid16,
                                   et::stream_t stream = nullptr) {
        if (pack_producer) {
            etChk(et_linear_bsr16_packed_resid_stats_f32(pack_producer.get(), et::f16(bias.get()), et::f16(input), nullptr,
                                                         et::f16(resid16), nullptr, nullptr, nullptr, V, stats, groups, size,
                                                         stream));
            return;
        }
        etChk(et_linear_bsr16_resid16_stats_f32(weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()),
                                                et::f16(bias.get()), et::f16(input), et::f16(resid16), V, stats, groups,
                                                size, (int)in_size, (int)out_size, stream));
    }
    // output = act(normalised(V) W^T + bias); fin_out, ln32, ln16 optional (null = not wanted)
    void forward_norm_f32in(half *output, const float *V, const float *stats, int groups, const half *gamma,
                            const half *beta, float eps, float *fin_out, float *ln32, half *ln16, int act,
                            et::stream_t stream = nullptr) {
        if (pack_consumer && !ln32 && !ln16) {
            etChk(et_norm_linear_bsr16_packed_f32in(pack_consumer.get(), V, stats, groups, et::f16(gamma), et::f16(beta), eps,
                                                    fin_out, et::f16(bias.get()), et::f16(output), size, act, stream));
            return;
        }
        etChk(et_norm_linear_bsr16_f32in(V, stats, groups, et::f16(gamma), et::f16(beta), eps, fin_out, ln32, et::f16(ln16),
                                         weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()),
                                         et::f16(bias.get()), et::f16(output), size, (int)in_size, (int)out_size, act,
                                         stream));
    }
    // ln_out = ln(src + skip); output = act(ln_out * W^T + bias) in one launch: the
    // SkipLayerNorm -> Linear -> activation sequence of Encoder/Encoder.h:85-89.  LN_t is
    // SkipLayerNorm (gamma(), beta(), epsilon(), width()).
    template <typename LN_t>
    void forward_skipln_act(half *output, half *ln_out, const half *src, const half *skip, const LN_t &ln,
                            int act, et::stream_t stream = nullptr) {
        et::require(ln.width() == (int)in_size, "Linear<tile_mat>: LayerNorm width must equal in_size");
        etChk(et_skipln_linear_bsr16_f16(et::f16(src), et::f16(skip), et::f16(ln.gamma()), et::f16(ln.beta()),
                                         ln.epsilon(), et::f16(ln_out), weight.row_ptr.get(),
                                         weight.row_offset.get(), et::f16(weight.data.get()),
                                         et::f16(bias.get()), et::f16(output), size, (int)in_size,
                                         (int)out_size, act, stream));
    }

    // `weight` is public, as in the reference, but what forward() multiplies with may be a copy made from it
    // when the object was built (the dense image, the streaming plan, the packs): a caller that writes into
    // weight.data, or replaces the structure, calls refresh() afterwards — outside any stream capture, it
    // allocates and synchronises — and every copy is made again, the role packs of the split normalisation
    // included.
    void refresh() {
        const bool had_producer = (bool)pack_producer, had_consumer = (bool)pack_consumer, had_heads = (bool)pack_heads;
        etChk(et_device_sync());  // launches still reading the old copies end first
        dense.reset();
        dense_out16.reset();
        plan.reset();
        pack.reset();
        pack_loop.reset();
        pack_producer.reset();
        pack_consumer.reset();
        pack_heads.reset();
        check();
        if (had_producer) prepare_split_producer(producer_nwave);
        if (had_consumer) prepare_split_consumer(consumer_nwave);
        if (had_heads) prepare_qkv_heads(heads_nhead, heads_gamma, heads_beta);
    }

  private:
    void check() {
        et::require(weight.blk_row_num * 16 == (int)out_size && weight.blk_col_num * 16 == (int)in_size,
                    "Linear<tile_mat>: weight shape does not match in/out sizes");
        et::require(bias.size == out_size, "Linear<tile_mat>: bias must hold out_size values");
        if (size > 0 && size % 16 == 0 && wants_dense((int)in_size, (int)out_size, weight.num_blk) &&
            !names_a_position_twice()) {
            dense = std::make_unique<et::DeviceBuffer<half>>((std::size_t)in_size * out_size);
            dense_out16 = std::make_unique<et::DeviceBuffer<half>>((std::size_t)size * out_size);  // forward allocates nothing
            etChk(et_bsr16_to_dense_f16(weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()),
                                        et::f16(dense->get()), (int)in_size, (int)out_size, nullptr));
            etChk(et_device_sync());
            return;
        }
        if (size > 0 && size % 16 == 0 && wants_plan((int)in_size, size)) {
            et_bsr_plan p = nullptr;
            etChk(et_bsr16_plan_create(weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()), size,
                                       (int)in_size, (int)out_size, 0, 0, 0, &p));
            plan.reset(p);
            return;
        }
        if (size <= kPlainPackMaxRows) pack = make_pack(0);
        if (size >= kRowLoopMinRows && in_size <= 1536) {
            pack_loop = make_pack(ET_PACK_ROW_LOOP, 0, 1 << 30);
            int mt = 0, groups = 0;
            if (pack_loop) etChk(et_bsr16_pack_info(pack_loop.get(), &mt, &groups, nullptr, nullptr, nullptr));
            if (pack_loop && (long)((size + mt * 16 - 1) / (mt * 16)) * groups < 256) pack_loop.reset();  // the chip would idle
        }
    }
    // a pack for this weight and `size` rows, or null where the packed kernel does not apply
    pack_ptr make_pack(int flags, int nwave = 0, int max_rows = kPackMaxRows) const {
        pack_ptr made;
        if (!packed_enabled() || size <= 0 || size % 16 != 0 || size > max_rows || in_size % 128 != 0 || in_size > 4096)
            return made;
        if (flags != ET_PACK_ROW_LOOP && !pack_pays()) return made;
        et_bsr_pack p = nullptr;
        const int s = et_bsr16_pack_create(weight.row_ptr.get(), weight.row_offset.get(), et::f16(weight.data.get()), size,
                                           (int)in_size, (int)out_size, flags, nwave, &p);
        if (s == ET_ERR_UNSUPPORTED) return made;  // the unpacked kernel keeps the shape
        etChk(s);
        made.reset(p);
        return made;
    }
    // true when some block-row lists one column twice, or an index lies outside the matrix (such a
    // weight stays with the tile kernel, which reports it)
    bool names_a_position_twice() const {
        const std::vector<int> rp = weight.row_ptr.to_host(), col = weight.row_offset.to_host();
        std::vector<char> seen((std::size_t)weight.blk_col_num);
        for (int r = 0; r + 1 < (int)rp.size(); r++) {
            if (rp[r] < 0 || rp[r + 1] < rp[r] || rp[r + 1] > (int)col.size()) return true;
            std::fill(seen.begin(), seen.end(), 0);
            for (int t = rp[r]; t < rp[r + 1]; t++) {
                if (col[t] < 0 || col[t] >= weight.blk_col_num || seen[(std::size_t)col[t]]) return true;
                seen[(std::size_t)col[t]] = 1;
            }
        }
        return false;
    }
};

// unstructured CSR — Linear/Linear.h:88-112, Linear/cusp.cu:23-82.  Single non-zeros give a
// matrix core nothing to skip, and the scalar CSR kernel (et_linear_csr_f16) is 10-25 times slower
// than the dense GEMM at 80-95 % sparsity.  Where the shapes allow the GEMM (token rows and both
// widths multiples of 16) and at least kDenseFromDensity of the elements are non-zero, the
// constructor therefore sums the non-zeros into a dense image on the host (duplicates of one
// position add up, as they do in the sparse product) and forward multiplies with that; sparser
// or odd-shaped weights stay on the CSR kernel.
template <> class Linear<csr_mat> {
  public:
    static constexpr double kDenseFromDensity = 0.02;
    const uint32_t in_size;
    const uint32_t out_size;
    const int size;
    std::unique_ptr<et::DeviceBuffer<int>> indptr;
    std::unique_ptr<et::DeviceBuffer<int>> indices;
    std::unique_ptr<et::DeviceBuffer<half>> data;
    std::unique_ptr<et::DeviceBuffer<half>> dense;  // [out x in] image, or empty
    et::DeviceBuffer<half> bias;

    Linear(int _in_size, int _out_size, const csr_mat &w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), size(_size), bias(b, (std::size_t)_out_size) {
        et::require(w.nrow == _out_size && w.ncol == _in_size, "Linear<csr_mat>: weight shape mismatch");
        // both paths below (the dense image and the CSR kernel, which indexes its LDS strip with the
        // column ids) rely on a consistent structure
        et::fmt::validate_csr(w.indptr, w.indices, w.data.size(), w.nrow, w.ncol);
        std::vector<half> h(w.data.size());
        for (std::size_t i = 0; i < h.size(); i++) h[i] = static_cast<half>(w.data[i]);
        indptr = std::make_unique<et::DeviceBuffer<int>>(w.indptr);
        indices = std::make_unique<et::DeviceBuffer<int>>(w.indices);
        data = std::make_unique<et::DeviceBuffer<half>>(h);
        const double cells = (double)_in_size * (double)_out_size;
        if (_size % 16 == 0 && _in_size % 16 == 0 && _out_size % 16 == 0 && _size > 0 &&
            (double)w.data.size() >= kDenseFromDensity * cells) {
            std::vector<float> img((std::size_t)_in_size * (std::size_t)_out_size, 0.0f);
            for (int r = 0; r < _out_size; r++)
                for (int k = w.indptr[(std::size_t)r]; k < w.indptr[(std::size_t)r + 1]; k++) {
                    const int c = w.indices[(std::size_t)k];
                    et::require(c >= 0 && c < _in_size, "Linear<csr_mat>: column index out of range");
                    // the value as the CSR kernel sees it: rounded to binary16 first
                    img[(std::size_t)r * (std::size_t)_in_size + (std::size_t)c] += static_cast<float>(h[(std::size_t)k]);
                }
            std::vector<half> himg(img.size());
            for (std::size_t i = 0; i < img.size(); i++) himg[i] = static_cast<half>(img[i]);
            dense = std::make_unique<et::DeviceBuffer<half>>(himg);
        }
    }
    Linear(Linear<csr_mat> &&other) = default;
    void forward(half *output, const half *input, et::stream_t stream = nullptr) {
        forward_act(output, input, ET_ACT_NONE, stream);
    }
    void forward_act(half *output, const half *input, int act, et::stream_t stream = nullptr) {
        if (dense) {
            etChk(et_linear_dense_f16(et::f16(dense->get()), et::f16(bias.get()), et::f16(input), et::f16(output),
                                      size, (int)in_size, (int)out_size, act, stream));
            return;
        }
        etChk(et_linear_csr_f16(indptr->get(), indices->get(), et::f16(data->get()), et::f16(bias.get()),
                                et::f16(input), et::f16(output), size, (int)in_size, (int)out_size, act,
                                stream));
    }
};

// 1x16 vector pruning — Linear/Linear.h:153-167 (the reference's kernel is a stub,
// Linear/SPMM1x16.cu:35-124; this one computes y = x W^T + b).  A matrix core multiplies whole
// 16x16 cells and up to about 95 % vector sparsity nearly every cell holds a vector, so no
// product can be skipped: the weight is expanded to its dense image once, on the device, and
// forward runs the dense GEMM on it (et_linear_vec1x16_f16 works on the vectors directly and
// is 3-5 times slower at 80 %).
template <> class Linear<mat1x16> {
  public:
    const uint32_t in_size;
    const uint32_t out_size;
    const int size;
    mat1x16 weight;
    et::DeviceBuffer<half> bias;
    et::DeviceBuffer<half> dense;  // [out x in] image of weight

    Linear(int _in_size, int _out_size, const mat1x16 &w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), size(_size), weight(w), bias(b, (std::size_t)_out_size),
          dense((std::size_t)_in_size * (std::size_t)_out_size) {
        expand();
    }
    Linear(int _in_size, int _out_size, mat1x16 &&w, const half *b, int _size)
        : in_size(_in_size), out_size(_out_size), size(_size), weight(std::move(w)),
          bias(b, (std::size_t)_out_size), dense((std::size_t)_in_size * (std::size_t)_out_size) {
        expand();
    }
    void forward(half *output, const half *input, et::stream_t stream = nullptr) {
        forward_act(output, input, ET_ACT_NONE, stream);
    }
    void forward_act(half *output, const half *input, int act, et::stream_t stream = nullptr) {
        etChk(et_linear_dense_f16(et::f16(dense.get()), et::f16(bias.get()), et::f16(input), et::f16(output),
                                  size, (int)in_size, (int)out_size, act, stream));
    }

  private:
    void expand() {
        etChk(et_vec1x16_to_dense_f16(weight.tile_idx.get(), weight.row_idx.get(), et::f16(weight.data.get()),
                                      et::f16(dense.get()), (int)in_size, (int)out_size, nullptr));
        etChk(et_device_sync());
    }
};

#include "gen_linear.hpp"

namespace et {

// binary32 output of any Linear: its own forward_f32 where the container's kernel can store
// the accumulator unrounded (tile_mat), else the binary16 result widened (one rounding of the
// projection's output; the residual stream it is added to stays binary32 either way).
template <typename L, typename = void> struct has_forward_f32 : std::false_type {};
template <typename L>
struct has_forward_f32<L, std::void_t<decltype(std::declval<L &>().forward_f32(
                              static_cast<float *>(nullptr), static_cast<const half *>(nullptr),
                              static_cast<stream_t>(nullptr)))>> : std::true_type {};

template <typename L>
void linear_forward_f32(L &lin, float *out32, const half *in, half *scratch16, stream_t stream) {
    if constexpr (has_forward_f32<L>::value) {
        lin.forward_f32(out32, in, stream);
    } else {
        lin.forward(scratch16, in, stream);
        etChk(et_f16_to_f32(out32, f16(scratch16), (std::size_t)lin.size * (std::size_t)lin.out_size, stream));
    }
}

}  // namespace et
