// The sweeps the reference measures with, written against the class layer
// (include/et/*.h) the way the reference's own drivers are:
//
//   et_sweeps linear <in> <out> <seq>         sparsity 0, 0.05 … 0.95 for the dense, column-,
//                                             row- and tile-pruned Linear (Linear/test/benchmark.cu:13-57)
//   et_sweeps seqlen                          attention block, seq 16 … 512 step 16, model
//                                             {768, 768, seq, 12, 4096, 768} (test/Attention/test_seqlen.cu:11-52)
//   et_sweeps table2 <nlayer> <sparsity>...   N encoder layers, uniform tile pruning and the
//                                             attention-aware configuration (test/Table2/main.cu:22-45,
//                                             test/Table2/template.hpp:13-118)
//   et_sweeps concurrent <in> <out> <seq> <sparsity>
//                                             three tile-pruned Linears on one stream and on three
//                                             (Linear/test/test_concurrent.cu)
//
// Times are microseconds per forward, launches back to back with one device
// synchronisation at the end (wtime_new, lib/wtime.h:22-35), after one warm-up.
// Output: one line per series, "name v0 v1 ...", so a plot script can read it.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <string>
#include <vector>

#include "et/Encoder.h"
#include "et/wtime.h"

using model_para_t = std::shared_ptr<Model_t>;

static void print_series(const std::string &name, const std::vector<double> &v) {
    std::cout << name;
    for (double x : v) std::printf(" %.3f", x);
    std::cout << std::endl;
}

// ---- Linear/test/benchmark.cu ---------------------------------------------------
template <typename mat_t> static std::vector<double> linear_sparsity_sweep(int in_size, int out_size, int seq_len) {
    std::vector<double> res;
    et::DeviceBuffer<half> IN((std::size_t)seq_len * in_size, half_one);
    et::DeviceBuffer<half> OUT((std::size_t)out_size * seq_len);
    for (int i = 0; i < 20; i++) {
        const float sparsity = 0.05f * i;
        auto layer = gen_sparse_linear<mat_t>(out_size, in_size, seq_len, sparsity);
        layer->forward(OUT.get(), IN.get());
        etChk(et_device_sync());
        res.push_back(wtime_new(
            50, [&]() { layer->forward(OUT.get(), IN.get()); }, []() { etChk(et_device_sync()); }));
    }
    return res;
}

static int run_linear(int in_size, int out_size, int seq_len) {
    std::printf("# Linear forward, in %d out %d rows %d; columns: sparsity 0.00 .. 0.95 step 0.05; us\n", in_size,
                out_size, seq_len);
    print_series("base_mat", linear_sparsity_sweep<base_mat>(in_size, out_size, seq_len));
    print_series("col_mat", linear_sparsity_sweep<col_mat>(in_size, out_size, seq_len));
    print_series("row_mat", linear_sparsity_sweep<row_mat>(in_size, out_size, seq_len));
    print_series("tile_mat", linear_sparsity_sweep<tile_mat>(in_size, out_size, seq_len));
    return 0;
}

// ---- test/Attention/test_seqlen.cu ----------------------------------------------
template <typename attn_tag> static std::vector<double> attention_seqlen_sweep() {
    using w_mat_t = base_mat;
    using attn_config = Attention_config<w_mat_t, w_mat_t, w_mat_t, w_mat_t, attn_tag>;
    constexpr float sparsity = 0.6f;  // dense weights ignore it, as in the reference driver
    std::vector<double> res;
    for (int seq_len = 16; seq_len <= 512; seq_len += 16) {
        auto para = std::make_shared<Model_t>(Model_t{768, 768, seq_len, 12, 4096, 768});
        et::DeviceBuffer<half> IN((std::size_t)para->emdim * seq_len, static_cast<half>(0.2f));
        et::DeviceBuffer<half> OUT((std::size_t)para->emdim * seq_len);
        auto LQ = gen_sparse_linear<w_mat_t>(para->kdim, para->emdim, seq_len, sparsity);
        auto LK = gen_sparse_linear<w_mat_t>(para->kdim, para->emdim, seq_len, sparsity);
        auto LV = gen_sparse_linear<w_mat_t>(para->vdim, para->emdim, seq_len, sparsity);
        auto LO = gen_sparse_linear<w_mat_t>(para->emdim, para->vdim, seq_len, sparsity);
        Attention<attn_config> attn(std::move(LQ), std::move(LK), std::move(LV), std::move(LO), para);
        attn.forward(OUT.get(), IN.get(), IN.get(), IN.get());
        etChk(et_device_sync());
        res.push_back(wtime_new(
            50, [&]() { attn.forward(OUT.get(), IN.get(), IN.get(), IN.get()); }, []() { etChk(et_device_sync()); }));
    }
    return res;
}

static int run_seqlen() {
    std::printf("# attention block (Q, K, V, O dense 768x768, 12 heads); columns: seq 16 .. 512 step 16; us\n");
    print_series("OTF_attn_full", attention_seqlen_sweep<OTF_attn_full>());
    print_series("OTF_attn_sharedQK", attention_seqlen_sweep<OTF_attn_sharedQK>());
    print_series("Norm_attn", attention_seqlen_sweep<Norm_attn>());
    return 0;
}

// ---- test/Table2 ----------------------------------------------------------------
struct layer_times {
    double eager;     // launches issued one by one, as the reference's driver does
    double replayed;  // the same launches recorded once in a graph and replayed
};

template <typename encoder_t>
static layer_times time_layers(std::vector<std::unique_ptr<encoder_t>> &model, model_para_t para) {
    et::DeviceBuffer<half> IN((std::size_t)para->emdim * para->seq_len, static_cast<half>(0.2f));
    et::DeviceBuffer<half> OUT((std::size_t)para->emdim * para->seq_len);
    for (auto &layer : model) layer->forward(OUT.get(), IN.get());
    etChk(et_device_sync());
    layer_times t;
    t.eager = wtime_new(
        50,
        [&]() {
            for (auto &layer : model) layer->forward(OUT.get(), IN.get());
        },
        []() { etChk(et_device_sync()); });
    et_stream stream = nullptr;
    et_graph graph = nullptr;
    etChk(et_stream_create(&stream));
    etChk(et_graph_begin_capture(stream));
    for (auto &layer : model) layer->forward(OUT.get(), IN.get(), stream);
    etChk(et_graph_end_capture(stream, &graph));
    etChk(et_graph_launch(graph, stream));
    etChk(et_stream_sync(stream));
    t.replayed = wtime_new(
        50, [&]() { etChk(et_graph_launch(graph, stream)); }, [&]() { etChk(et_stream_sync(stream)); });
    etChk(et_graph_destroy(graph));
    etChk(et_stream_destroy(stream));
    return t;
}

// every matrix of the layer pruned in tiles at one sparsity (template.hpp:13-52)
static layer_times test_uniform_tile(model_para_t para, float sparsity, int nlayer) {
    using mat_t = tile_mat;
    using attn_config = Attention_config<mat_t, mat_t, mat_t, mat_t, OTF_attn_full, true, false>;
    using encoder_config = Encoder_config<attn_config, mat_t, mat_t, GELU_OP>;
    std::vector<std::unique_ptr<Encoder<encoder_config>>> model((std::size_t)nlayer);
    for (auto &layer : model) {
        auto LQKV = gen_sparse_linear<mat_t>(para->kdim * 2 + para->vdim, para->emdim, para->seq_len, sparsity);
        auto LO = gen_sparse_linear<mat_t>(para->emdim, para->vdim, para->seq_len, sparsity);
        auto attn = std::make_unique<Attention<attn_config>>(std::move(LQKV), std::move(LO), para);
        auto L1 = gen_sparse_linear<mat_t>(para->dimFF, para->emdim, para->seq_len, sparsity);
        auto L2 = gen_sparse_linear<mat_t>(para->emdim, para->dimFF, para->seq_len, sparsity);
        layer = std::make_unique<Encoder<encoder_config>>(std::move(attn), gen_skLN(para->emdim), gen_skLN(para->emdim),
                                                          std::move(L1), std::move(L2), para);
    }
    return time_layers(model, para);
}

// attention-aware: W_V row-pruned, compact V, the rest tile-pruned (template.hpp:78-118)
static layer_times test_prune_attn(model_para_t para, float sparsity, int nlayer) {
    using attn_config = Attention_config<tile_mat, tile_mat, row_mat, tile_mat, Prune_attn, false, true>;
    using encoder_config = Encoder_config<attn_config, tile_mat, tile_mat, GELU_OP>;
    std::vector<std::unique_ptr<Encoder<encoder_config>>> model((std::size_t)nlayer);
    for (auto &layer : model) {
        auto LQ = gen_sparse_linear<tile_mat>(para->kdim, para->emdim, para->seq_len, sparsity);
        auto LK = gen_sparse_linear<tile_mat>(para->kdim, para->emdim, para->seq_len, sparsity);
        auto LV = gen_sparse_linear<row_mat>(para->vdim, para->emdim, para->seq_len, sparsity);
        auto LO = gen_sparse_linear<tile_mat>(para->emdim, para->vdim, para->seq_len, sparsity);
        auto attn = std::make_unique<Attention<attn_config>>(std::move(LQ), std::move(LK), std::move(LV), std::move(LO),
                                                            para);
        auto L1 = gen_sparse_linear<tile_mat>(para->dimFF, para->emdim, para->seq_len, sparsity);
        auto L2 = gen_sparse_linear<tile_mat>(para->emdim, para->dimFF, para->seq_len, sparsity);
        layer = std::make_unique<Encoder<encoder_config>>(std::move(attn), gen_skLN(para->emdim), gen_skLN(para->emdim),
                                                          std::move(L1), std::move(L2), para);
    }
    return time_layers(model, para);
}

static int run_table2(int nlayer, const std::vector<float> &sparsities) {
    auto para = std::make_shared<Model_t>(Model_t{768, 768, 128, 12, 768 * 4, 768});
    std::printf("# %d encoder layers, seq 128, hidden 768, FFN 3072; columns: sparsity", nlayer);
    for (float sp : sparsities) std::printf(" %.2f", sp);
    std::printf("; ms per forward of all layers\n");
    std::vector<double> tile, aware, tile_graph, aware_graph;
    for (float sp : sparsities) {
        const layer_times t = test_uniform_tile(para, sp, nlayer), a = test_prune_attn(para, sp, nlayer);
        tile.push_back(t.eager / 1000);
        aware.push_back(a.eager / 1000);
        tile_graph.push_back(t.replayed / 1000);
        aware_graph.push_back(a.replayed / 1000);
    }
    print_series("tile", tile);
    print_series("aware", aware);
    print_series("tile_graph", tile_graph);
    print_series("aware_graph", aware_graph);
    return 0;
}

// ---- Linear/test/test_concurrent.cu ---------------------------------------------
static int run_concurrent(int in_size, int out_size, int seq_len, float sparsity) {
    std::vector<std::unique_ptr<Linear<tile_mat>>> layers;
    std::vector<et::DeviceBuffer<half>> outs;
    for (int i = 0; i < 3; i++) {
        layers.push_back(gen_sparse_linear<tile_mat>(out_size, in_size, seq_len, sparsity));
        outs.emplace_back((std::size_t)out_size * seq_len);
    }
    et::DeviceBuffer<half> IN((std::size_t)seq_len * in_size, half_one);
    et_stream streams[3];
    for (auto &s : streams) etChk(et_stream_create(&s));
    auto one_stream = [&]() {
        for (int i = 0; i < 3; i++) layers[i]->forward(outs[i].get(), IN.get());
    };
    auto three_streams = [&]() {
        for (int i = 0; i < 3; i++) layers[i]->forward(outs[i].get(), IN.get(), streams[i]);
    };
    one_stream();
    three_streams();
    etChk(et_device_sync());
    const double serial = wtime_new(50, one_stream, []() { etChk(et_device_sync()); });
    const double parallel = wtime_new(50, three_streams, []() { etChk(et_device_sync()); });
    for (auto &s : streams) etChk(et_stream_destroy(s));
    std::printf("# three tile-pruned Linears, in %d out %d rows %d sparsity %.2f; us per group of three\n", in_size,
                out_size, seq_len, sparsity);
    print_series("one_stream", {serial});
    print_series("three_streams", {parallel});
    return 0;
}

static int usage() {
    std::puts("usage: et_sweeps linear <in> <out> <seq> | seqlen | table2 <nlayer> <sparsity>... | "
              "concurrent <in> <out> <seq> <sparsity>");
    return 2;
}

int main(int ac, char **av) {
    if (ac < 2) return usage();
    const std::string mode = av[1];
    try {
        if (mode == "linear" && ac == 5) return run_linear(std::atoi(av[2]), std::atoi(av[3]), std::atoi(av[4]));
        if (mode == "seqlen") return run_seqlen();
        if (mode == "table2" && ac >= 4) {
            std::vector<float> sp;
            for (int i = 3; i < ac; i++) sp.push_back((float)std::atof(av[i]));
            return run_table2(std::atoi(av[2]), sp);
        }
        if (mode == "concurrent" && ac == 6)
            return run_concurrent(std::atoi(av[2]), std::atoi(av[3]), std::atoi(av[4]), (float)std::atof(av[5]));
    } catch (const et::Error &e) {
        std::fprintf(stderr, "et_sweeps: %s\n", e.what());
        return 1;
    }
    return usage();
}
