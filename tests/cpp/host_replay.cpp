// Replays, without a GPU, the host side of what the encoder-stack tests do through the C ABI:
// tile patterns from the format generators, et_model_create, et_model_set_*, et_model_finalize,
// forwards (graph and eager), changed lengths and masks, single layers, the archive loader and
// the error paths.  Built by tests/test_host_sanitized.py together with host/*.cpp and host
// stand-ins for the device entry points, all under AddressSanitizer and
// UndefinedBehaviorSanitizer: any read or write outside a buffer on these paths ends the run.
//
//   host_replay [directory with weights.txt + archives of a 2-layer H128 nh2 FF256 model]
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <filesystem>
#include <fstream>
#include <iterator>
#include <string>
#include <vector>

#include "et_abi.h"

namespace {

int g_failures = 0;

#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            fprintf(stderr, "host_replay: %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            g_failures++;                                                   \
        }                                                                   \
    } while (0)

#define OK(call)                                                                              \
    do {                                                                                      \
        int s_ = (call);                                                                      \
        if (s_ != ET_OK) {                                                                    \
            fprintf(stderr, "host_replay: %s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, s_, \
                    et_last_error());                                                         \
            g_failures++;                                                                     \
        }                                                                                     \
    } while (0)

struct Weight {
    int out, in;
    std::vector<int32_t> row_ptr, col;
    std::vector<et_f16> tiles, bias;
};

// Arrays are sized exactly (no slack), so that an over-read of one element is out of bounds.
Weight make_weight(int out, int in, float sparsity, uint64_t seed) {
    Weight w;
    w.out = out;
    w.in = in;
    int ntile = et_fmt_kept_count((int64_t)(out / 16) * (in / 16), sparsity);
    w.row_ptr.resize((size_t)out / 16 + 1);
    w.col.resize((size_t)ntile);
    OK(et_fmt_tile_pattern(out, in, sparsity, seed, w.row_ptr.data(), w.col.data(), &ntile));
    EXPECT((int)w.col.size() == ntile);
    w.tiles.assign((size_t)ntile * 256, (et_f16)0x2000);
    w.bias.assign((size_t)out, (et_f16)0x1000);
    return w;
}

struct Case {
    int H, nh, FF, S, B, nlayer;
    float sparsity;
    int act, use_graph;
    bool lens;
    int mixed = 0;
};

void run_case(const Case &c, uint64_t seed) {
    et_model_desc d{};
    d.kdim = d.vdim = d.emdim = c.H;
    d.seq_len = c.S;
    d.nhead = c.nh;
    d.dimFF = c.FF;
    d.nlayer = c.nlayer;
    d.batch = c.B;
    d.act = c.act;
    d.eps = 1e-5f;
    d.use_graph = c.use_graph;
    d.mixed = c.mixed;
    et_model m = nullptr;
    OK(et_model_create(&d, &m));
    if (!m) return;
    std::vector<et_f16> gamma((size_t)c.H, 0x3C00), beta((size_t)c.H, 0);
    for (int l = 0; l < c.nlayer; l++) {
        const int dims[4][2] = {{3 * c.H, c.H}, {c.H, c.H}, {c.FF, c.H}, {c.H, c.FF}};
        for (int w = 0; w < 4; w++) {
            Weight bw = make_weight(dims[w][0], dims[w][1], c.sparsity, seed + 10 * (uint64_t)l + (uint64_t)w);
            OK(et_model_set_bsr16_f16(m, l, w, bw.row_ptr.data(), bw.col.data(), bw.tiles.data(),
                                      (int)bw.col.size(), bw.bias.data()));
        }
        OK(et_model_set_norm_f16(m, l, 0, gamma.data(), beta.data()));
        OK(et_model_set_norm_f16(m, l, 1, gamma.data(), beta.data()));
    }
    std::vector<int32_t> lens((size_t)c.B);
    for (int b = 0; b < c.B; b++) lens[(size_t)b] = c.S / 2 + b % (c.S / 2);
    if (c.lens) OK(et_model_set_lens(m, lens.data()));
    OK(et_model_finalize(m));
    const size_t bytes = (size_t)c.B * c.S * c.H * sizeof(et_f16);
    void *in = nullptr, *out = nullptr, *out2 = nullptr;
    OK(et_malloc(&in, bytes));
    OK(et_malloc(&out, bytes));
    OK(et_malloc(&out2, bytes));
    for (int rep = 0; rep < 3; rep++) OK(et_model_forward(m, (et_f16 *)out, (const et_f16 *)in, nullptr));
    OK(et_model_forward(m, (et_f16 *)out2, (const et_f16 *)in, nullptr));  // other buffers: recapture
    OK(et_model_forward(m, (et_f16 *)out2, (const et_f16 *)out2, nullptr)); // in place
    OK(et_model_set_lens(m, lens.data()));
    OK(et_model_forward(m, (et_f16 *)out, (const et_f16 *)in, nullptr));
    std::vector<et_f16> mask((size_t)c.S * c.S, 0);
    OK(et_model_set_mask(m, mask.data()));
    OK(et_model_forward(m, (et_f16 *)out, (const et_f16 *)in, nullptr));
    OK(et_model_set_mask(m, nullptr));
    OK(et_model_set_lens(m, nullptr));
    for (int l = 0; l < c.nlayer; l++)
        OK(et_model_forward_layer(m, l, (et_f16 *)(l % 2 ? out : out2), (const et_f16 *)(l % 2 ? out2 : out), nullptr));
    OK(et_model_sync(m));
    OK(et_model_destroy(m));
    OK(et_free(in));
    OK(et_free(out));
    OK(et_free(out2));
}

void error_paths() {
    et_model_desc d{};
    d.kdim = d.vdim = d.emdim = 128;
    d.seq_len = 32;
    d.nhead = 2;
    d.dimFF = 256;
    d.nlayer = 1;
    d.batch = 1;
    d.act = ET_ACT_GELU;
    et_model m = nullptr;
    OK(et_model_create(&d, &m));
    EXPECT(et_model_finalize(m) != ET_OK);  // nothing set
    const std::vector<int32_t> row_ptr = {0, 1, 2, 3, 4, 5, 6, 7, 9};  // back() != ntile
    const std::vector<int32_t> col(8, 0);
    const std::vector<et_f16> tiles(8 * 256, 0);
    EXPECT(et_model_set_bsr16_f16(m, 0, ET_W_O, row_ptr.data(), col.data(), tiles.data(), 8, nullptr) != ET_OK);
    std::vector<int32_t> bad_col(8, 0), good_ptr = {0, 1, 2, 3, 4, 5, 6, 7, 8};
    bad_col[5] = -5;
    EXPECT(et_model_set_bsr16_f16(m, 0, ET_W_O, good_ptr.data(), bad_col.data(), tiles.data(), 8, nullptr) != ET_OK);
    bad_col[5] = 8;
    EXPECT(et_model_set_bsr16_f16(m, 0, ET_W_O, good_ptr.data(), bad_col.data(), tiles.data(), 8, nullptr) != ET_OK);
    const std::vector<et_f16> g(128, 0x3C00);
    EXPECT(et_model_set_norm_f16(m, 3, 0, g.data(), g.data()) != ET_OK);
    OK(et_model_destroy(m));
    et_model none = nullptr;
    EXPECT(et_model_load("/nonexistent/weights.txt", "/nonexistent/", &d, &none) != ET_OK);
    EXPECT(none == nullptr);
    d.kdim = d.vdim = d.emdim = 100;
    d.nhead = 3;
    EXPECT(et_model_create(&d, &none) != ET_OK);
}

void load_archives(const std::string &dir) {
    et_model_desc d{};
    d.kdim = d.vdim = d.emdim = 128;
    d.seq_len = 32;
    d.nhead = 2;
    d.dimFF = 256;
    d.nlayer = 2;
    d.batch = 1;
    d.act = ET_ACT_GELU;
    d.use_graph = 1;
    et_model m = nullptr;
    OK(et_model_load((dir + "/weights.txt").c_str(), (dir + "/").c_str(), &d, &m));
    if (!m) return;
    void *in = nullptr, *out = nullptr;
    OK(et_malloc(&in, 32 * 128 * 2));
    OK(et_malloc(&out, 32 * 128 * 2));
    OK(et_model_forward(m, (et_f16 *)out, (const et_f16 *)in, nullptr));
    OK(et_model_destroy(m));
    OK(et_free(in));
    OK(et_free(out));
}

// Damaged archives must be refused with a status, never read out of bounds: the first archive
// of the model is truncated at many lengths and has single bytes of its zip directory, local
// header and npy header overwritten; every variant goes through et_model_load.
void corrupt_archives(const std::string &dir) {
    namespace fs = std::filesystem;
    const fs::path work = fs::path(dir) / "damaged";
    fs::create_directories(work);
    for (const auto &e : fs::directory_iterator(dir))
        if (e.is_regular_file()) fs::copy_file(e.path(), work / e.path().filename(), fs::copy_options::overwrite_existing);
    std::ifstream list((work / "weights.txt").string());
    std::string first;
    std::getline(list, first);
    const fs::path victim = work / first;
    std::ifstream in(victim.string(), std::ios::binary);
    const std::vector<char> good((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    EXPECT(good.size() > 200);
    et_model_desc d{};
    d.kdim = d.vdim = d.emdim = 128;
    d.seq_len = 32;
    d.nhead = 2;
    d.dimFF = 256;
    d.nlayer = 2;
    d.batch = 1;
    d.act = ET_ACT_GELU;
    int refused = 0, tried = 0;
    auto attempt = [&](const std::vector<char> &bytes) {
        std::ofstream out(victim.string(), std::ios::binary | std::ios::trunc);
        out.write(bytes.data(), (std::streamsize)bytes.size());
        out.close();
        et_model m = nullptr;
        const int s = et_model_load((work / "weights.txt").string().c_str(), (work.string() + "/").c_str(), &d, &m);
        tried++;
        if (s != ET_OK) refused++;
        if (m) OK(et_model_destroy(m));
    };
    for (std::size_t cut : {std::size_t(0), std::size_t(10), std::size_t(21), std::size_t(22), std::size_t(45), good.size() / 3,
                            good.size() / 2, good.size() - 100, good.size() - 23, good.size() - 22, good.size() - 1})
        attempt(std::vector<char>(good.begin(), good.begin() + (std::ptrdiff_t)std::min(cut, good.size())));
    uint64_t rng = 0x9E3779B97F4A7C15ull;
    for (int k = 0; k < 400; k++) {
        rng = rng * 6364136223846793005ull + 1442695040888963407ull;
        std::vector<char> bad = good;
        // half of the hits in the last 400 bytes (central directory and end record), the rest anywhere
        const std::size_t span = (k & 1) ? std::min<std::size_t>(400, bad.size()) : bad.size();
        const std::size_t pos = bad.size() - 1 - (std::size_t)((rng >> 20) % span);
        bad[pos] = (char)(rng >> 56);
        if (k % 5 == 0) bad[(pos + 1) % bad.size()] = (char)0xFF;
        attempt(bad);
    }
    EXPECT(refused >= 11);  // every truncation at least; damaged payload bytes may still load
    printf("host_replay: %d damaged archives, %d refused\n", tried, refused);
}

}  // namespace

int main(int argc, char **argv) {
    const Case cases[] = {
        {128, 2, 256, 32, 2, 2, 0.5f, ET_ACT_GELU, 1, true},    // two-layer stack, graph
        {128, 2, 256, 32, 2, 2, 0.5f, ET_ACT_GELU, 0, true},    // eager
        {128, 2, 256, 32, 2, 1, 0.5f, ET_ACT_GELU, 1, false},   // recapture for new buffers and lengths
        {256, 4, 512, 48, 1, 3, 0.7f, ET_ACT_RELU, 1, false},   // layer by layer (QKV: 230 tiles)
        {768, 12, 3072, 128, 8, 2, 0.8f, ET_ACT_GELU, 1, false},  // headline shape, two layers
        {128, 2, 256, 32, 2, 3, 0.5f, ET_ACT_GELU, 1, true, 1},    // mixed precision, graph
        {256, 4, 512, 48, 1, 1, 0.7f, ET_ACT_RELU, 0, false, 1},   // mixed precision, one layer, eager
    };
    uint64_t seed = 4000;
    for (const Case &c : cases) run_case(c, seed += 100);
    error_paths();
    if (argc > 1) {
        load_archives(argv[1]);
        corrupt_archives(argv[1]);
    }
    if (g_failures) {
        fprintf(stderr, "host_replay: %d check(s) failed\n", g_failures);
        return 1;
    }
    printf("host_replay ok\n");
    return 0;
}
