// Drives the C++ class layer (include/et/*.h) the way the reference's own
// programs do, and writes the results as .npy files for the pytest side to
// compare with the CPU oracle.  Usage:  class_layer_cases <case> <dir>
//   example       two ReLU encoder layers + a decoder Linear loaded from weights.txt/.npz,
//                 the model assembly of the reference example (example/main.cu:24-182)
//   prune_attn    Attention<tile, tile, row_mat, tile, Prune_attn> (attention-aware pruning)
//   fused_attn    FusedAttention<NOTF_fused_attn> with the W_VO built by et::build_vo_weight
//   fused_otf     FusedAttention<OTF_fused_attn>: the same attention with the probabilities kept on chip
//   fused_prune   FusedAttention<NOTF_fused_prune_attn> over a column-pruned W_VO
//   factories     the gen_* test factories: closed forms of the reference drivers
//   attn_variants Attention<> with separate Q/K/V projections under the tags OTF_attn_full,
//                 OTF_attn_full_mixed, OTF_attn_Ofused (tile-sparse) and Norm_attn (dense)
//   encoder_fuse  Encoder_fuse<NOTF_fused_attn> (pre-computed VO attention + tile-sparse FFN), in both
//                 the all-fp16 and the mixed-precision form
//   file_ctors    row_mat / col_mat / csr_mat built from their raw files
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <iostream>
#include <string>

#include "et/Encoder.h"
#include "et/weights.hpp"
#include "et/wtime.h"

using et::npy::npy_load;
using et::npy::npy_save;

static std::vector<half> load_half(const std::string &path) {
    auto a = npy_load(path);
    return vec_F2H(a.as_vector<float>());
}
static void save_half(const std::string &path, const et::DeviceBuffer<half> &buf, std::size_t rows, std::size_t cols) {
    std::vector<half> h = buf.to_host();
    std::vector<float> f(h.size());
    for (std::size_t i = 0; i < h.size(); i++) f[i] = static_cast<float>(h[i]);
    npy_save(path, f.data(), "<f4", 4, {rows, cols});
}
static std::vector<int> load_int(const std::string &path) { return npy_load(path).as_vector<int>(); }
static std::vector<int> read_meta(const std::string &dir) { return load_int(dir + "/meta.npy"); }

static tile_mat tile_from(Weights &w, const std::string &name, int in) {
    return tile_mat(w.load_mat<int>("row_ptr", name), w.load_mat<int>("column", name),
                    vec_F2H(w.load_mat<float>("data", name)), in / 16);
}

// ---- example/main.cu ------------------------------------------------------------
static int run_example(const std::string &dir) {
    using mat_t = tile_mat;
    using attn_config = Attention_config<mat_t, mat_t, mat_t, mat_t, OTF_attn_full, true, false>;
    using encoder_config = Encoder_config<attn_config, mat_t, mat_t, RELU_OP>;
    const auto meta = read_meta(dir);  // kdim vdim seq nhead dimFF emdim nlayer batch decoder_width
    auto para = std::make_shared<Model_t>(Model_t{meta[0], meta[1], meta[2], meta[3], meta[4], meta[5], meta[6]});
    const int batch = meta[7], text = meta[8];
    const int rows = batch * para->seq_len;
    Weights weights(dir + "/weights.txt", dir + "/");
    std::vector<std::unique_ptr<Encoder<encoder_config>>> model((std::size_t)para->nlayer);
    for (int l = 0; l < para->nlayer; l++) {
        const std::string pre = "transformer_encoder.layers." + std::to_string(l) + ".";
        const auto QKVname = pre + "self_attn.in_proj_.npz";
        et::DeviceBuffer<half> BQKV(vec_F2H(weights.load_mat<float>("B", QKVname)));
        auto LQKV = std::make_unique<Linear<mat_t>>(para->emdim, para->kdim * 3, tile_from(weights, QKVname, para->emdim),
                                                    BQKV, rows);
        const auto Oname = pre + "self_attn.out_proj..npz";
        et::DeviceBuffer<half> BO(vec_F2H(weights.load_mat<float>("B", Oname)));
        auto LO = std::make_unique<Linear<mat_t>>(para->vdim, para->emdim, tile_from(weights, Oname, para->vdim), BO, rows);
        auto attn = std::make_unique<Attention<attn_config>>(std::move(LQKV), std::move(LO), para, batch);
        const auto LN1name = pre + "norm1..npz", LN2name = pre + "norm2..npz";
        auto LN1 = std::make_unique<SkipLayerNorm>(vec_F2H(weights.load_mat<float>("W", LN1name)).data(),
                                                   vec_F2H(weights.load_mat<float>("B", LN1name)).data(), para->emdim);
        auto LN2 = std::make_unique<SkipLayerNorm>(vec_F2H(weights.load_mat<float>("W", LN2name)).data(),
                                                   vec_F2H(weights.load_mat<float>("B", LN2name)).data(), para->emdim);
        const auto L1name = pre + "linear1..npz", L2name = pre + "linear2..npz";
        et::DeviceBuffer<half> BL1(vec_F2H(weights.load_mat<float>("B", L1name)));
        auto L1 = std::make_unique<Linear<mat_t>>(para->emdim, para->dimFF, tile_from(weights, L1name, para->emdim), BL1, rows);
        et::DeviceBuffer<half> BL2(vec_F2H(weights.load_mat<float>("B", L2name)));
        auto L2 = std::make_unique<Linear<mat_t>>(para->dimFF, para->emdim, tile_from(weights, L2name, para->dimFF), BL2, rows);
        model[(std::size_t)l] = std::make_unique<Encoder<encoder_config>>(std::move(attn), std::move(LN1), std::move(LN2),
                                                                          std::move(L1), std::move(L2), para);
    }
    const auto Dname = std::string("decoder..npz");
    et::DeviceBuffer<half> BD(vec_F2H(weights.load_mat<float>("B", Dname)));
    auto LD = std::make_unique<Linear<mat_t>>(para->emdim, text, tile_from(weights, Dname, para->emdim), BD, rows);

    et::DeviceBuffer<half> IN(load_half(dir + "/input.npy"));
    et::DeviceBuffer<half> A((std::size_t)rows * para->emdim), B((std::size_t)rows * para->emdim);
    et::DeviceBuffer<half> OUT((std::size_t)rows * text);
    half *src = IN.get();
    for (int l = 0; l < para->nlayer; l++) {
        half *dst = (l % 2 == 0) ? A.get() : B.get();
        model[(std::size_t)l]->forward(dst, src);
        src = dst;
    }
    LD->forward(OUT.get(), src);
    etChk(et_device_sync());
    save_half(dir + "/out.npy", OUT, (std::size_t)rows, (std::size_t)text);
    save_half(dir + "/hidden.npy", (para->nlayer % 2 == 1) ? A : B, (std::size_t)rows, (std::size_t)para->emdim);
    // the reference's timing protocol on the same objects (lib/wtime.h:22-35)
    const double us = wtime_new(
        20, [&]() { model[0]->forward(A.get(), IN.get()); }, []() { etChk(et_device_sync()); });
    std::printf("encoder layer forward: %.1f us\n", us);
    return 0;
}

// ---- attention-aware pruning (test/Table2/template.hpp:56-97) -------------------
static int run_prune_attn(const std::string &dir) {
    using attn_config = Attention_config<tile_mat, tile_mat, row_mat, tile_mat, Prune_attn, false, true>;
    const auto meta = read_meta(dir);  // H seq nhead batch
    const int H = meta[0], S = meta[1], nh = meta[2], batch = meta[3], rows = batch * S;
    auto para = std::make_shared<Model_t>(Model_t{H, H, S, nh, 4 * H, H, 1});
    auto dense_tile_linear = [&](const std::string &tag) {
        auto W = npy_load(dir + "/W" + tag + ".npy").as_vector<float>();
        auto b = load_half(dir + "/b" + tag + ".npy");
        return std::make_unique<Linear<tile_mat>>(H, H, tile_mat::from_dense(W.data(), H, H), b.data(), rows);
    };
    auto LQ = dense_tile_linear("q"), LK = dense_tile_linear("k"), LO = dense_tile_linear("o");
    auto row_id = load_int(dir + "/v_row_id.npy");
    auto v_rows = load_half(dir + "/v_rows.npy");
    auto bv = load_half(dir + "/bv.npy");
    row_mat WV(et::DeviceBuffer<int>(row_id), et::DeviceBuffer<half>(v_rows), H, H);
    auto LV = std::make_unique<Linear<row_mat>>(H, H, std::move(WV), bv.data(), rows);
    Attention<attn_config> attn(std::move(LQ), std::move(LK), std::move(LV), std::move(LO), para, batch);
    auto lens = load_int(dir + "/lens.npy");
    attn.set_lens(lens.data());
    et::DeviceBuffer<half> X(load_half(dir + "/input.npy")), OUT((std::size_t)rows * H);
    attn.forward(OUT.get(), X.get(), X.get(), X.get());
    etChk(et_device_sync());
    save_half(dir + "/out.npy", OUT, (std::size_t)rows, (std::size_t)H);
    return 0;
}

// ---- pre-computed VO attention (Fused_attention/test/testfused.cu:17-97) --------
template <typename tag> static int run_fused(const std::string &dir) {
    using attn_config = Attention_config<base_mat, base_mat, base_mat, base_mat, tag, false, true>;
    const auto meta = read_meta(dir);  // H seq nhead batch
    const int H = meta[0], S = meta[1], nh = meta[2], batch = meta[3], rows = batch * S;
    auto para = std::make_shared<Model_t>(Model_t{H, H, S, nh, 4 * H, H, 1});
    auto dense_linear = [&](const std::string &tag2) {
        auto W = load_half(dir + "/W" + tag2 + ".npy");
        auto b = load_half(dir + "/b" + tag2 + ".npy");
        return std::make_unique<Linear<base_mat>>(H, H, base_mat(W), b.data(), rows);
    };
    auto LQ = dense_linear("q"), LK = dense_linear("k");
    auto Wv = npy_load(dir + "/Wv.npy").as_vector<float>(), bv = npy_load(dir + "/bv.npy").as_vector<float>();
    auto Wo = npy_load(dir + "/Wo.npy").as_vector<float>();
    std::vector<float> Wvo, bvo;
    et::build_vo_weight(Wv.data(), bv.data(), Wo.data(), H, H, H, nh, Wvo, bvo);
    et::DeviceBuffer<half> biasO(load_half(dir + "/bo.npy"));
    et::DeviceBuffer<half> X(load_half(dir + "/input.npy")), OUT((std::size_t)rows * H);
    auto lens = load_int(dir + "/lens.npy");
    if constexpr (std::is_same<tag, NOTF_fused_prune_attn>::value) {
        auto col_id = load_int(dir + "/vo_col_id.npy");
        const std::size_t N = col_id.size();
        std::vector<half> Wc((std::size_t)nh * H * N), bc((std::size_t)nh * N);
        for (int h = 0; h < nh; h++) {
            for (int i = 0; i < H; i++)
                for (std::size_t j = 0; j < N; j++)
                    Wc[((std::size_t)h * H + i) * N + j] = static_cast<half>(Wvo[((std::size_t)h * H + i) * H + col_id[j]]);
            for (std::size_t j = 0; j < N; j++) bc[(std::size_t)h * N + j] = static_cast<half>(bvo[(std::size_t)h * H + col_id[j]]);
        }
        col_mat W(et::DeviceBuffer<int>(col_id), et::DeviceBuffer<half>(Wc), nh * H, H, (int)N);
        auto LVO = std::make_unique<Linear_VO_prune>(W, et::DeviceBuffer<half>(bc), para);
        FusedAttention<attn_config> attn(std::move(LQ), std::move(LK), std::move(LVO), biasO, para, batch);
        attn.set_lens(lens.data());
        attn.forward(OUT.get(), X.get(), X.get(), X.get());
    } else {
        auto LVO = std::make_unique<Linear_VO>(et::DeviceBuffer<half>(vec_F2H(Wvo)), et::DeviceBuffer<half>(vec_F2H(bvo)), para);
        FusedAttention<attn_config> attn(std::move(LQ), std::move(LK), std::move(LVO), biasO, para, batch);
        attn.set_lens(lens.data());
        attn.forward(OUT.get(), X.get(), X.get(), X.get());
    }
    etChk(et_device_sync());
    save_half(dir + "/out.npy", OUT, (std::size_t)rows, (std::size_t)H);
    // the offline W_VO builder's result, for the test to check against numpy
    npy_save(dir + "/Wvo.npy", Wvo.data(), "<f4", 4, {(std::size_t)nh, (std::size_t)H, (std::size_t)H});
    npy_save(dir + "/bvo.npy", bvo.data(), "<f4", 4, {(std::size_t)nh, (std::size_t)H});
    return 0;
}

// ---- gen_* factories: closed forms of the reference drivers ---------------------
static float first_value(const et::DeviceBuffer<half> &b, std::size_t i = 0) { return static_cast<float>(b.to_host()[i]); }

static int run_factories(const std::string &dir) {
    std::vector<float> out;
    const int T = 64;
    et::DeviceBuffer<half> X1024((std::size_t)T * 1024, half_one), Y((std::size_t)T * 1024);
    // dense ones: in_size * 1 + 0.5 (Linear/test/test_cublas.cu:12-19), at a width fp16 holds exactly
    et::DeviceBuffer<half> X256((std::size_t)T * 256, half_one);
    gen_dense_linear<base_mat>(128, 256, T)->forward(Y.get(), X256.get());
    out.push_back(first_value(Y, 5));                                   // 256.5
    gen_dense_linear<tile_mat>(128, 256, T)->forward(Y.get(), X256.get());
    out.push_back(first_value(Y, 5));                                   // 256.5
    // tile-sparse ones: 16 * tiles_in_block_row + 0.5 (Linear/test/test_tile.cu:56-75)
    {
        auto lin = gen_sparse_linear<tile_mat>(128, 256, T, 0.5f);
        lin->forward(Y.get(), X256.get());
        auto rp = lin->weight.row_ptr.to_host();
        out.push_back(first_value(Y, 0));
        out.push_back(16.0f * (float)(rp[1] - rp[0]) + 0.5f);          // expected for block-row 0
        out.push_back((float)lin->weight.num_blk);                     // 64 of 128 tiles
    }
    gen_dense_linear<row_mat>(128, 256, T)->forward(Y.get(), X256.get());
    out.push_back(first_value(Y, 7));                                   // 256.5
    {
        auto lin = gen_sparse_linear<row_mat>(128, 256, T, 0.5f);      // 64 live rows: x.w + b, others b alone
        lin->forward(Y.get(), X256.get());
        auto ids = lin->weight.row_id->to_host();
        auto y = Y.to_host();
        out.push_back(static_cast<float>(y[(std::size_t)ids[0]]));       // 256.5
        int dead = 0;
        while (std::find(ids.begin(), ids.end(), dead) != ids.end()) dead++;
        out.push_back(static_cast<float>(y[(std::size_t)dead]));         // 0.5
        out.push_back((float)ids.size());                                // 64
    }
    {
        auto lin = gen_sparse_linear<col_mat>(128, 256, T, 0.5f);      // 128 live inputs, weights 0.5
        lin->forward(Y.get(), X256.get());
        out.push_back(first_value(Y, 3));                               // 128 * 0.5 + 0.5 = 64.5
    }
    gen_dense_linear<csr_mat>(128, 256, T)->forward(Y.get(), X256.get());
    out.push_back(first_value(Y, 9));                                   // 256.5
    gen_dense_linear<mat1x16>(128, 256, T)->forward(Y.get(), X256.get());
    out.push_back(first_value(Y, 11));                                  // 256.5
    // Linear_VO with weight 0.2, bias 0.2, input ones over 1024 features: 0.2*1024 + 0.2 = 205.0
    // (Fused_attention/test/testVO.cu:10-16; the fp16 result is 205.0 exactly)
    {
        auto para = std::make_shared<Model_t>(Model_t{1024, 1024, 64, 16, 4096, 1024, 1});
        const half p2 = static_cast<half>(0.2f);
        Linear_VO vo(et::DeviceBuffer<half>((std::size_t)16 * 1024 * 1024, p2), et::DeviceBuffer<half>((std::size_t)16 * 1024, p2), para);
        et::DeviceBuffer<half> VO((std::size_t)16 * 64 * 1024);
        vo.forward(VO.get(), X1024.get());
        etChk(et_device_sync());
        out.push_back(first_value(VO, 12345));
    }
    // SkipLayerNorm test instance: gamma = beta = 0.2; a constant row normalises to beta
    {
        auto ln = gen_skLN(768);
        et::DeviceBuffer<half> A((std::size_t)T * 768, static_cast<half>(0.7f)), B((std::size_t)T * 768, static_cast<half>(0.1f)),
            O((std::size_t)T * 768);
        ln->forward(O.get(), A.get(), B.get(), T);
        out.push_back(first_value(O, 100));                             // 0.2
    }
    // Linear<csr_mat> multiplies with a dense image from 2 % density on and with the CSR kernel below:
    // both against a direct call of the CSR kernel (weights and inputs are ones: sums are exact)
    for (float sp : {0.8f, 0.99f}) {
        auto lin = gen_sparse_linear<csr_mat>(128, 256, T, sp);
        lin->forward(Y.get(), X256.get());
        et::DeviceBuffer<half> Y2((std::size_t)T * 128);
        etChk(et_linear_csr_f16(lin->indptr->get(), lin->indices->get(), et::f16(lin->data->get()), et::f16(lin->bias.get()),
                                et::f16(X256.get()), et::f16(Y2.get()), T, 256, 128, ET_ACT_NONE, nullptr));
        etChk(et_device_sync());
        auto a = Y.to_host(), b = Y2.to_host();
        bool same = true;
        for (std::size_t i = 0; i < (std::size_t)T * 128; i++) same = same && static_cast<float>(a[i]) == static_cast<float>(b[i]);
        out.push_back(same ? 1.0f : 0.0f);
        out.push_back(lin->dense ? 1.0f : 0.0f);  // 1 at 80 %, 0 at 99 %
    }
    // DeviceBuffer value semantics: deep copy, move, clear, set
    {
        et::DeviceBuffer<half> a(8, static_cast<half>(3.0f));
        et::DeviceBuffer<half> b(a);
        a.set(static_cast<half>(4.0f));
        out.push_back(first_value(b));                                  // 3 (deep copy)
        et::DeviceBuffer<half> c(std::move(a));
        out.push_back(first_value(c));                                  // 4
        c.clear();
        out.push_back(first_value(c));                                  // 0
        out.push_back((float)(a.get() == nullptr));                     // 1: moved-from
        // the pointer constructor takes device memory as well as host memory (lib/CUDA_ptr.hpp:18-31)
        et::DeviceBuffer<half> src(8, static_cast<half>(7.0f));
        et::DeviceBuffer<half> from_dev(src.get(), 8);
        src.set(static_cast<half>(1.0f));
        out.push_back(first_value(from_dev, 5));                        // 7 (copied, not aliased)
        const std::vector<half> host8(8, static_cast<half>(6.0f));
        et::DeviceBuffer<half> from_host(host8.data(), 8);
        out.push_back(first_value(from_host, 5));                       // 6
    }
    {
        // Linear<tile_mat> multiplies with a copy of its weight made at construction; a caller that writes
        // into weight.data calls refresh().  All tiles set to 2: 32 * tiles_in_block_row + 0.5
        auto lin = gen_sparse_linear<tile_mat>(128, 256, T, 0.5f);
        lin->forward(Y.get(), X256.get());
        etChk(et_device_sync());
        lin->weight.data.set(static_cast<half>(2.0f));
        lin->refresh();
        lin->forward(Y.get(), X256.get());
        auto rp = lin->weight.row_ptr.to_host();
        out.push_back(first_value(Y, 0));
        out.push_back(32.0f * (float)(rp[1] - rp[0]) + 0.5f);
    }
    etChk(et_device_sync());
    // Linear<row_mat> picks its form by the share of features that survive: half of them -> a dense image of the
    // weight; one in sixteen -> the scattering GEMM behind a fill.  Both: live features x.w + b, dead ones b.
    for (const float sp : {0.5f, 0.9375f}) {
        auto lin = gen_sparse_linear<row_mat>(512, 256, T, sp);
        lin->forward(Y.get(), X256.get());
        auto ids = lin->weight.row_id->to_host();
        auto y = Y.to_host();
        int dead = 0;
        while (std::find(ids.begin(), ids.end(), dead) != ids.end()) dead++;
        out.push_back(static_cast<float>(y[(std::size_t)ids[0]]));             // 256.5
        out.push_back(static_cast<float>(y[(std::size_t)dead]));               // 0.5
        out.push_back(static_cast<float>(y[(std::size_t)(T - 1) * 512 + (std::size_t)ids.back()]));  // 256.5, last row
        out.push_back((float)ids.size());                                      // 256, 32
        out.push_back(lin->dense_image ? 1.0f : 0.0f);                         // 1, 0
    }
    npy_save(dir + "/factories.npy", out.data(), "<f4", 4, {out.size()});
    return 0;
}

// ---- Attention<> with separate projections under every tag that has not been built elsewhere ------
template <typename MAT, typename tag>
static void run_attn_variant(const std::string &dir, const std::string &out_name, bool as_f32 = false) {
    using attn_config = Attention_config<MAT, MAT, MAT, MAT, tag, false, true>;
    const auto meta = read_meta(dir);  // H seq nhead batch
    const int H = meta[0], S = meta[1], nh = meta[2], batch = meta[3], rows = batch * S;
    auto para = std::make_shared<Model_t>(Model_t{H, H, S, nh, 4 * H, H, 1});
    auto make = [&](const std::string &t) {
        auto b = load_half(dir + "/b" + t + ".npy");
        if constexpr (std::is_same<MAT, tile_mat>::value) {
            auto W = npy_load(dir + "/W" + t + ".npy").as_vector<float>();
            return std::make_unique<Linear<tile_mat>>(H, H, tile_mat::from_dense(W.data(), H, H), b.data(), rows);
        } else {
            auto W = load_half(dir + "/W" + t + ".npy");
            return std::make_unique<Linear<base_mat>>(H, H, base_mat(W), b.data(), rows);
        }
    };
    Attention<attn_config> attn(make("q"), make("k"), make("v"), make("o"), para, batch);
    auto lens = load_int(dir + "/lens.npy");
    attn.set_lens(lens.data());
    et::DeviceBuffer<half> X(load_half(dir + "/input.npy")), OUT((std::size_t)rows * H);
    if (as_f32) {
        if constexpr (!std::is_same<tag, OTF_attn_Ofused>::value) {
            et::DeviceBuffer<float> OUT32((std::size_t)rows * H);
            et::DeviceBuffer<half> scratch((std::size_t)rows * H);
            attn.forward_f32(OUT32.get(), X.get(), X.get(), X.get(), scratch.get());
            etChk(et_device_sync());
            auto f = OUT32.to_host();
            npy_save(dir + "/" + out_name, f.data(), "<f4", 4, {(std::size_t)rows, (std::size_t)H});
        }
        return;
    }
    attn.forward(OUT.get(), X.get(), X.get(), X.get());
    etChk(et_device_sync());
    save_half(dir + "/" + out_name, OUT, (std::size_t)rows, (std::size_t)H);
}

static int run_attn_variants(const std::string &dir) {
    run_attn_variant<tile_mat, OTF_attn_full>(dir, "out_full.npy");
    run_attn_variant<tile_mat, OTF_attn_full_mixed>(dir, "out_full_mixed.npy");
    run_attn_variant<tile_mat, OTF_attn_Ofused>(dir, "out_ofused.npy");
    run_attn_variant<tile_mat, OTF_attn>(dir, "out_otf.npy");
    run_attn_variant<base_mat, Norm_attn>(dir, "out_norm.npy");
    run_attn_variant<tile_mat, OTF_attn_full>(dir, "out_full_f32.npy", true);   // binary32 output projection
    run_attn_variant<base_mat, OTF_attn_full>(dir, "out_dense_f32.npy", true);  // widened binary16 projection
    // the free function of Attention/kernel_fuseO.h:6-9 called directly on Q = K = V = input
    {
        const auto meta = read_meta(dir);
        const int H = meta[0], S = meta[1], nh = meta[2], batch = meta[3], rows = batch * S;
        auto para = std::make_shared<Model_t>(Model_t{H, H, S, nh, 4 * H, H, 1});
        auto Wo = npy_load(dir + "/Wo.npy").as_vector<float>();
        tile_mat wo = tile_mat::from_dense(Wo.data(), H, H);
        et::DeviceBuffer<half> bo(load_half(dir + "/bo.npy"));
        et::DeviceBuffer<half> X(load_half(dir + "/input.npy")), Z((std::size_t)rows * H), OUT((std::size_t)rows * H);
        et::AttnRun run;
        run.batch = batch;
        Multihead_atttion_fuseO(X.get(), X.get(), X.get(), nullptr, Z.get(), wo.row_ptr.get(), wo.row_offset.get(),
                                wo.data.get(), bo.get(), para, OUT.get(), run);
        etChk(et_device_sync());
        save_half(dir + "/out_fuseO_free.npy", OUT, (std::size_t)rows, (std::size_t)H);
        // ... and as one launch
        et::DeviceBuffer<half> Z1((std::size_t)rows * H), OUT1((std::size_t)rows * H);
        run.one_launch = true;
        Multihead_atttion_fuseO(X.get(), X.get(), X.get(), nullptr, Z1.get(), wo.row_ptr.get(), wo.row_offset.get(),
                                wo.data.get(), bo.get(), para, OUT1.get(), run);
        etChk(et_device_sync());
        save_half(dir + "/out_fuseO_one_launch.npy", OUT1, (std::size_t)rows, (std::size_t)H);
    }
    return 0;
}

// ---- Encoder_fuse (Encoder/Encoder.h:99-139) ------------------------------------------------------
static int run_encoder_fuse(const std::string &dir) {
    using attn_config = Attention_config<base_mat, base_mat, base_mat, base_mat, NOTF_fused_attn, false, true>;
    const auto meta = read_meta(dir);  // H seq nhead batch FF
    const int H = meta[0], S = meta[1], nh = meta[2], batch = meta[3], FF = meta[4], rows = batch * S;
    auto para = std::make_shared<Model_t>(Model_t{H, H, S, nh, FF, H, 1});
    auto build = [&]() {
        auto dense_linear = [&](const std::string &t) {
            auto W = load_half(dir + "/W" + t + ".npy");
            auto b = load_half(dir + "/b" + t + ".npy");
            return std::make_unique<Linear<base_mat>>(H, H, base_mat(W), b.data(), rows);
        };
        auto Wv = npy_load(dir + "/Wv.npy").as_vector<float>(), bv = npy_load(dir + "/bv.npy").as_vector<float>();
        auto Wo = npy_load(dir + "/Wo.npy").as_vector<float>();
        std::vector<float> Wvo, bvo;
        et::build_vo_weight(Wv.data(), bv.data(), Wo.data(), H, H, H, nh, Wvo, bvo);
        auto LVO = std::make_unique<Linear_VO>(et::DeviceBuffer<half>(vec_F2H(Wvo)), et::DeviceBuffer<half>(vec_F2H(bvo)), para);
        et::DeviceBuffer<half> biasO(load_half(dir + "/bo.npy"));
        auto attn = std::make_unique<FusedAttention<attn_config>>(dense_linear("q"), dense_linear("k"), std::move(LVO), biasO,
                                                                 para, batch);
        auto lens = load_int(dir + "/lens.npy");
        attn->set_lens(lens.data());
        auto ln = [&](const std::string &t) {
            return std::make_unique<SkipLayerNorm>(load_half(dir + "/g" + t + ".npy").data(),
                                                   load_half(dir + "/be" + t + ".npy").data(), H);
        };
        auto W1 = npy_load(dir + "/W1.npy").as_vector<float>(), W2 = npy_load(dir + "/W2.npy").as_vector<float>();
        auto L1 = std::make_unique<Linear<tile_mat>>(H, FF, tile_mat::from_dense(W1.data(), FF, H),
                                                     load_half(dir + "/b1.npy").data(), rows);
        auto L2 = std::make_unique<Linear<tile_mat>>(FF, H, tile_mat::from_dense(W2.data(), H, FF),
                                                     load_half(dir + "/b2.npy").data(), rows);
        return std::make_unique<Encoder_fuse<attn_config>>(std::move(attn), ln("1"), ln("2"), std::move(L1), std::move(L2),
                                                           para);
    };
    auto enc = build();
    et::DeviceBuffer<half> X(load_half(dir + "/input.npy")), OUT((std::size_t)rows * H);
    enc->forward_f16(OUT.get(), X.get());  // every activation binary16, as the reference stores them
    etChk(et_device_sync());
    save_half(dir + "/out.npy", OUT, (std::size_t)rows, (std::size_t)H);
    enc->forward(OUT.get(), X.get());  // the drop-in entry: binary32 residual stream inside the layer
    etChk(et_device_sync());
    save_half(dir + "/out_forward.npy", OUT, (std::size_t)rows, (std::size_t)H);
    // mixed precision: binary32 residual stream around the same sublayers
    enc->enable_mixed();
    et::DeviceBuffer<float> X32((std::size_t)rows * H), OUT32((std::size_t)rows * H);
    etChk(et_f16_to_f32(X32.get(), et::f16(X.get()), (std::size_t)rows * H, nullptr));
    enc->forward_mixed(OUT32.get(), OUT.get(), X32.get(), X.get());
    etChk(et_device_sync());
    auto f = OUT32.to_host();
    npy_save(dir + "/out_mixed32.npy", f.data(), "<f4", 4, {(std::size_t)rows, (std::size_t)H});
    save_half(dir + "/out_mixed16.npy", OUT, (std::size_t)rows, (std::size_t)H);
    return 0;
}

// ---- raw-file constructors (row_mat.hpp:15-29, col_mat.hpp:22-36, csr_mat.h:19-35) ------------------
static int run_file_ctors(const std::string &dir) {
    auto save_ints = [&](const std::string &name, const std::vector<int> &v) {
        npy_save(dir + "/" + name, v.data(), "<i4", 4, {v.size()});
    };
    auto save_halfs = [&](const std::string &name, const std::vector<half> &h) {
        std::vector<float> f(h.size());
        for (std::size_t i = 0; i < h.size(); i++) f[i] = static_cast<float>(h[i]);
        npy_save(dir + "/" + name, f.data(), "<f4", 4, {f.size()});
    };
    row_mat r(dir + "/small.row");
    save_ints("row_meta.npy", {r.nrow, r.ncol, r.nnz_row()});
    save_ints("row_id.npy", r.row_id->to_host());
    save_halfs("rows.npy", r.rows->to_host());
    col_mat c(dir + "/small.col");
    save_ints("col_meta.npy", {c.nrow, c.ncol, c.nnz_col, c.ldm});
    save_ints("col_id.npy", c.col_id->to_host());
    save_halfs("cols.npy", c.cols->to_host());
    csr_mat m(dir + "/small.csr");
    save_ints("csr_meta.npy", {m.nrow, m.ncol, m.nnz});
    save_ints("csr_indptr.npy", m.indptr);
    save_ints("csr_indices.npy", m.indices);
    npy_save(dir + "/csr_data.npy", m.data.data(), "<f4", 4, {m.data.size()});
    // damaged headers are refused
    int refused = 0;
    for (const char *name : {"/bad.row", "/bad.col", "/bad.csr"}) {
        try {
            if (std::string(name) == "/bad.row") row_mat bad(dir + name);
            else if (std::string(name) == "/bad.col") col_mat bad(dir + name);
            else csr_mat bad(dir + name);
        } catch (const et::Error &e) {
            if (e.status() == ET_ERR_IO) refused++;
        }
    }
    save_ints("refused.npy", {refused});
    return 0;
}

int main(int argc, char **argv) {
    if (argc < 3) {
        std::fprintf(stderr, "usage: %s <case> <dir>\n", argv[0]);
        return 2;
    }
    const std::string which = argv[1], dir = argv[2];
    try {
        if (which == "example") return run_example(dir);
        if (which == "prune_attn") return run_prune_attn(dir);
        if (which == "fused_attn") return run_fused<NOTF_fused_attn>(dir);
        if (which == "fused_otf") return run_fused<OTF_fused_attn>(dir);
        if (which == "fused_prune") return run_fused<NOTF_fused_prune_attn>(dir);
        if (which == "factories") return run_factories(dir);
        if (which == "attn_variants") return run_attn_variants(dir);
        if (which == "encoder_fuse") return run_encoder_fuse(dir);
        if (which == "file_ctors") return run_file_ctors(dir);
        std::fprintf(stderr, "unknown case %s\n", which.c_str());
        return 2;
    } catch (const et::Error &e) {
        std::fprintf(stderr, "et::Error %d: %s\n", e.status(), e.what());
        return 1;
    }
}
