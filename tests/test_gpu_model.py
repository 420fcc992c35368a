"""GPU parity of the encoder-stack handle (et_model_*), i.e. of the C++ class layer
(Linear / Attention / SkipLayerNorm / Encoder) it is built from, against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import formats as F
from tests import harness as Hn

pytestmark = pytest.mark.gpu

TOL_F16 = 2e-2  # fp16 path with fp32 accumulation


def run_model(et, m, x, reps=1):
    T, H = x.shape
    d_in = et.DeviceBuffer.from_numpy(x)
    d_out = et.DeviceBuffer.empty((T, H), np.float16)
    outs = []
    for _ in range(reps):
        et.check(et.lib().et_fill_f16(d_out.ptr, T * H, 0x7E00, None))
        et.sync()
        m.forward(d_out, d_in)
        m.sync()
        outs.append(d_out.numpy())
    return outs


@pytest.mark.parametrize("use_graph", [True, False])
def test_two_layer_stack_small(et, use_graph):
    H, nh, FF, S, B = 128, 2, 256, 32, 2
    layers = [Hn.LayerWeights(H, nh, FF, 0.5, seed=20 + i) for i in range(2)]
    lens = np.array([20, 32], np.int32)
    m = Hn.build_model(et, layers, S, B, lens=lens, use_graph=use_graph)
    x = Hn.randn((B * S, H), 99)
    outs = run_model(et, m, x, reps=3)
    want = Hn.oracle_stack(x, layers, B, lens)
    for o in outs:  # every graph replay equals the oracle (and hence the eager pass)
        assert Hn.max_abs(o, want) <= TOL_F16
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[1], outs[2])


def test_graph_recaptures_for_new_buffers_and_new_lens(et):
    H, nh, FF, S, B = 128, 2, 256, 32, 2
    layers = [Hn.LayerWeights(H, nh, FF, 0.5, seed=30)]
    m = Hn.build_model(et, layers, S, B)
    x1, x2 = Hn.randn((B * S, H), 1), Hn.randn((B * S, H), 2)
    o1 = run_model(et, m, x1)[0]
    o2 = run_model(et, m, x2)[0]  # other device buffers: the graph is captured again
    assert Hn.max_abs(o1, Hn.oracle_stack(x1, layers, B)) <= TOL_F16
    assert Hn.max_abs(o2, Hn.oracle_stack(x2, layers, B)) <= TOL_F16
    lens = np.array([7, 19], np.int32)
    m.set_lens(lens)
    o3 = run_model(et, m, x2)[0]
    assert Hn.max_abs(o3, Hn.oracle_stack(x2, layers, B, lens)) <= TOL_F16
    assert not np.array_equal(o2, o3)


def test_layer_by_layer_equals_stack(et):
    H, nh, FF, S, B = 256, 4, 512, 48, 1
    layers = [Hn.LayerWeights(H, nh, FF, 0.7, seed=40 + i) for i in range(3)]
    m = Hn.build_model(et, layers, S, B, act=1)
    x = Hn.randn((S, H), 3)
    full = run_model(et, m, x)[0]
    bufs = [et.DeviceBuffer.from_numpy(x), et.DeviceBuffer.empty((S, H), np.float16)]
    for i in range(3):
        m.forward_layer(i, bufs[(i + 1) % 2], bufs[i % 2])
    et.sync()
    assert np.array_equal(full, bufs[1].numpy(np.float16, (S, H)))
    assert Hn.max_abs(full, Hn.oracle_stack(x, layers, B, act="relu")) <= TOL_F16


def headline_layers(seed0):
    H, nh, FF = 768, 12, 3072
    return [Hn.LayerWeights(H, nh, FF, 0.8, seed=seed0 + i, attention_aware=0.25) for i in range(12)]


# Measured (max-abs over the [1024 x 768] output of layer 12, this workload, three seeds): the
# fp16-storage oracle is 1.8e-2 .. 2.3e-2 from the fp32 mathematics — rounding the residual stream
# to fp16 after every sublayer — and the mixed-precision oracle 6e-4 (4e-3 once the final result is
# rounded to fp16).  So the 2e-2 bound of the fp16 path against the fp32 CPU forward is a claim the
# mixed-precision mode can make with margin and the all-fp16 mode cannot make at this depth.
TOL_MIXED_VS_F32 = 1e-2      # mixed mode against the fp32 forward (half the north-star bound)
TOL_MIXED_VS_ORACLE = 6e-3   # against the oracle rounding where the engine does (one fp16 ulp at |x| <= 4 plus noise)
TOL_F16_DEEP = 5e-2          # all-fp16 storage over 12+ layers: two realisations of the storage noise


@pytest.mark.parametrize("seed0,xseed,mode", [(100, 4, 1), (300, 307, 1), (500, 507, 1), (100, 4, 2), (100, 4, 3),
                                               (300, 307, 3), (100, 4, 4), (300, 307, 4), (100, 4, 5)])
def test_bert_base_12_layers_batch8_tile80_attention_aware_mixed(et, seed0, xseed, mode):
    """The headline configuration in the engine's mixed-precision mode: 12 layers, B8 S128, 80 %
    tile sparsity, 25 % of the V rows (and the matching O columns) dead in head-aligned groups."""
    H, S, B = 768, 128, 8
    layers = headline_layers(seed0)
    assert len(layers[0].qkv.col_idx) == F.tile_count(3 * H, H, 0.8)
    m = Hn.build_model(et, layers, S, B, mixed=mode)
    x = Hn.randn((B * S, H), xseed)
    got = run_model(et, m, x, reps=2)
    want32 = Hn.oracle_stack(x, layers, B, store=None)
    want_mixed = Hn.oracle_stack(x, layers, B, store=torch.float16, resid=torch.float32)
    e32, em = Hn.max_abs(got[0], want32), Hn.max_abs(got[0], want_mixed)
    print(f"12-layer B8 S128 mixed (mode {mode}) seed {seed0}: vs fp32 forward {e32:.3e}, vs mixed oracle {em:.3e}")
    assert e32 <= TOL_MIXED_VS_F32 and em <= TOL_MIXED_VS_ORACLE
    assert np.array_equal(got[0], got[1])
    if mode in (1, 4):  # at this batch the engine takes the four-launch form by itself as well
        assert m.launches_per_layer() == 4, "the QKV projection did not move into the attention kernel"
    if mode == 5:
        assert m.launches_per_layer() == 5


@pytest.mark.parametrize("S,B,sp,padded,causal", [(128, 3, 0.8, True, False), (48, 5, 0.9, False, True),
                                                  (64, 9, 0.5, True, True), (16, 1, 0.95, False, False),
                                                  (128, 8, 0.8, True, False)])
def test_qkv_inside_attention_stacks(et, S, B, sp, padded, causal):
    """mixed = 4: the layers after the first project Q, K and V inside their attention kernel (768-wide models with
    heads of 64, sequences up to 128 tokens): padded, causal, short and odd batch counts, block-rows of few and of
    many tiles; against the oracle and against the five-launch form (the same arithmetic up to the order of the
    sums of the row statistics and one fused multiply-add in the normalisation)."""
    H, nh, FF = 768, 12, 512
    layers = [Hn.LayerWeights(H, nh, FF, sp, seed=900 + i) for i in range(3)]
    lens = np.random.default_rng(S * B).integers(S // 2, S + 1, B).astype(np.int32) if padded else None
    x = Hn.randn((B * S, H), 909)
    m4 = Hn.build_model(et, layers, S, B, lens=lens, causal=causal, mixed=4)
    m1 = Hn.build_model(et, layers, S, B, lens=lens, causal=causal, mixed=5)
    got4, got1 = run_model(et, m4, x, reps=3), run_model(et, m1, x, reps=1)
    assert m4.launches_per_layer() == 4 and m1.launches_per_layer() == 5
    want = Hn.oracle_stack(x, layers, B, lens, causal=causal, store=torch.float16, resid=torch.float32)
    a, b, c = got4[0].astype(np.float32), want.astype(np.float32), got1[0].astype(np.float32)
    if lens is not None:  # rows past a sequence's length are padding: not compared
        for i in range(B):
            for t in (a, b, c):
                t[i * S + lens[i]:(i + 1) * S] = 0
    print(f"QKV inside attention S={S} B={B} sparsity {sp}: vs oracle {Hn.max_abs(a, b):.3e}, vs five launches {Hn.max_abs(a, c):.3e}")
    # (against the other launch form: both results are binary16, one unit in the last place of a value in [4, 8) is 3.9e-3)
    assert Hn.max_abs(a, b) <= 4e-3 and Hn.max_abs(a, c) <= 8e-3
    assert np.array_equal(got4[0], got4[1]) and np.array_equal(got4[1], got4[2])


def test_qkv_inside_attention_chosen_by_batch(et):
    """mixed = 1 takes the four-launch form by itself where it measured faster (here 12 sequences of 64 tokens on 12
    heads, 8 as well) and keeps five launches elsewhere (4 sequences, 40 sequences)."""
    H, nh, FF, S = 768, 12, 512, 64
    layers = [Hn.LayerWeights(H, nh, FF, 0.8, seed=920 + i) for i in range(2)]
    for B, launches in ((12, 4), (8, 4), (4, 5), (40, 5)):
        m = Hn.build_model(et, layers, S, B, mixed=1)
        assert m.launches_per_layer() == launches
        x = Hn.randn((B * S, H), 929)
        got = run_model(et, m, x)[0]
        want = Hn.oracle_stack(x, layers, B, store=torch.float16, resid=torch.float32)
        assert Hn.max_abs(got, want) <= 4e-3


def test_qkv_inside_attention_falls_back(et):
    """Shapes the fused kernel does not take (here a 256-wide model) run mixed = 4 exactly as mixed = 1."""
    H, nh, FF, S, B = 256, 4, 512, 64, 2
    layers = [Hn.LayerWeights(H, nh, FF, 0.7, seed=940 + i) for i in range(2)]
    x = Hn.randn((B * S, H), 949)
    m4, m1 = Hn.build_model(et, layers, S, B, mixed=4), Hn.build_model(et, layers, S, B, mixed=1)
    assert m4.launches_per_layer() == 5
    assert np.array_equal(run_model(et, m4, x)[0], run_model(et, m1, x)[0])
    # the BERT-large shape (1024 wide, 512 tokens) is outside it as well
    layers, lens, x, S, B = bert_large_case(2)
    m4, m1 = Hn.build_model(et, layers, S, B, lens=lens, mixed=4), Hn.build_model(et, layers, S, B, lens=lens, mixed=1)
    assert m4.launches_per_layer() == 5
    assert np.array_equal(run_model(et, m4, x)[0], run_model(et, m1, x)[0])


def test_bert_base_12_layers_all_fp16_storage(et):
    """The same stack with every activation stored as fp16 (mixed = 0).  Checked layer by layer
    against the fp16-storage oracle: the first layers, where the two realisations of the rounding
    noise have not drifted apart, hold the per-layer bound; the full depth holds the loose one."""
    H, S, B = 768, 128, 8
    layers = headline_layers(100)
    x = Hn.randn((B * S, H), 4)
    for depth, tol in ((1, 4e-3), (2, TOL_F16), (12, TOL_F16_DEEP)):
        m = Hn.build_model(et, layers[:depth], S, B)
        got = run_model(et, m, x, reps=2)
        err = Hn.max_abs(got[0], Hn.oracle_stack(x, layers[:depth], B))
        print(f"{depth}-layer B8 S128 fp16 storage: vs fp16-storage oracle {err:.3e}")
        assert err <= tol
        assert np.array_equal(got[0], got[1])


def test_chain_launches_equal_separate_launches(et):
    """mixed = 3 runs everything between two attention kernels as one launch whose workgroups meet at
    counters in their XCD's L2 instead of at kernel boundaries: the same arithmetic on the same packs
    as mixed = 5 (five separate launches), so the results agree bit for bit, replay after replay; and the model reports that the
    chain really ran (two launches per layer)."""
    H, S, B = 768, 128, 8
    layers = headline_layers(700)
    x = Hn.randn((B * S, H), 707)
    m5 = Hn.build_model(et, layers, S, B, mixed=5)
    m2 = Hn.build_model(et, layers, S, B, mixed=3)
    a = run_model(et, m5, x, reps=2)
    b = run_model(et, m2, x, reps=4)
    assert m5.launches_per_layer() == 5
    assert m2.launches_per_layer() == 2, f"the chain was not taken: {et.lib().et_last_error().decode()}"
    for r in b:
        assert np.array_equal(r, a[0])


def test_bench_workload_mixed_precision(et):
    """Exactly the weights and input bench.py times (its own generator and seeds)."""
    import bench
    layers = bench.build_layers(et)
    m = bench.build_model(et, layers, use_graph=True)
    assert m.desc.mixed == 1 and m.launches_per_layer() == 4
    x = np.random.default_rng(4).standard_normal((bench.B * bench.S, bench.H), dtype=np.float32).astype(np.float16)
    got = run_model(et, m, x)[0]
    want32, want_mixed = bench.oracle_forwards(layers, x)
    e32, em = Hn.max_abs(got, want32), Hn.max_abs(got, want_mixed)
    print(f"bench workload mixed: vs fp32 forward {e32:.3e}, vs mixed oracle {em:.3e}")
    assert e32 <= TOL_MIXED_VS_F32 and em <= TOL_MIXED_VS_ORACLE


def bert_large_case(nlayer):
    H, nh, FF, S, B = 1024, 16, 4096, 512, 4
    layers = [Hn.LayerWeights(H, nh, FF, 0.9, seed=200 + i) for i in range(nlayer)]
    lens = torch.randint(256, 513, (B,), generator=Hn.rng(5)).numpy().astype(np.int32)
    return layers, lens, Hn.randn((B * S, H), 5), S, B


def test_bert_large_shape_padded_24_layers_mixed(et):
    """BERT-large shaped stack at its full depth: 24 layers, H1024, 16 heads, FFN 4096, S512, B4,
    90 % tiles, lengths in [256,512], fp16 matrix-core operands with fp32 softmax, LayerNorm and
    residual stream."""
    layers, lens, x, S, B = bert_large_case(24)
    m = Hn.build_model(et, layers, S, B, lens=lens, mixed=True)
    got = run_model(et, m, x)[0]
    want32 = Hn.oracle_stack(x, layers, B, lens, store=None)
    want_mixed = Hn.oracle_stack(x, layers, B, lens, store=torch.float16, resid=torch.float32)
    e32, em = Hn.max_abs(got, want32), Hn.max_abs(got, want_mixed)
    print(f"BERT-large shape, 24 layers, lens={lens.tolist()}: vs fp32 forward {e32:.3e}, vs mixed oracle {em:.3e}")
    assert e32 <= TOL_MIXED_VS_F32 and em <= TOL_MIXED_VS_ORACLE


def test_bert_large_shape_padded_4_layers_fp16_storage(et):
    """Four of those layers with all-fp16 storage against the fp16-storage oracle."""
    layers, lens, x, S, B = bert_large_case(4)
    m = Hn.build_model(et, layers, S, B, lens=lens)
    got = run_model(et, m, x)[0]
    err = Hn.max_abs(got, Hn.oracle_stack(x, layers, B, lens))
    print(f"BERT-large shape, 4 layers, fp16 storage: max-abs={err:.3e}")
    assert err <= TOL_F16


@pytest.mark.parametrize("mode", [1, 2])  # SkipLayerNorm folded into the projections / launched on its own
@pytest.mark.parametrize("use_graph", [True, False])
def test_mixed_small_stack_graph_eager_inplace_and_single_layers(et, use_graph, mode):
    H, nh, FF, S, B = 128, 2, 256, 32, 2
    layers = [Hn.LayerWeights(H, nh, FF, 0.5, seed=60 + i) for i in range(3)]
    lens = np.array([20, 32], np.int32)
    m = Hn.build_model(et, layers, S, B, lens=lens, use_graph=use_graph, mixed=mode)
    x = Hn.randn((B * S, H), 98)
    outs = run_model(et, m, x, reps=3)
    want = Hn.oracle_stack(x, layers, B, lens, store=torch.float16, resid=torch.float32)
    for o in outs:
        assert Hn.max_abs(o, want) <= 4e-3
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[1], outs[2])
    # in place: the graph's warm-up pass must not consume the input
    d = et.DeviceBuffer.from_numpy(x)
    m.forward(d, d)
    m.sync()
    assert np.array_equal(d.numpy(), outs[0])
    # layer by layer through fp16 buffers: each layer restarts its residual from fp16
    bufs = [et.DeviceBuffer.from_numpy(x), et.DeviceBuffer.empty((B * S, H), np.float16)]
    ref = Hn.f32(x)
    for i in range(3):
        m.forward_layer(i, bufs[(i + 1) % 2], bufs[i % 2])
        ref = Hn.f32(Hn.oracle_stack(ref.numpy(), layers[i:i + 1], B, lens, store=torch.float16,
                                     resid=torch.float32).astype(np.float16))
    et.sync()
    assert Hn.max_abs(bufs[1].numpy(np.float16, (B * S, H)), ref.numpy()) <= 4e-3


def _random_stack_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        nh = int(rng.integers(1, 9))
        hd = 16 * int(rng.integers(1, 5))
        cases.append((nh * hd, nh, 16 * int(rng.integers(2, 49)), 16 * int(rng.integers(1, 13)), int(rng.integers(1, 6)),
                      int(rng.integers(1, 4)), float(rng.choice([0.3, 0.6, 0.8, 0.9])), int(rng.integers(0, 3)),
                      bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), int(rng.integers(1, 1 << 20))))
    return cases


@pytest.mark.parametrize("H,nh,FF,S,B,nlayer,sp,mode,padded,causal,seed", _random_stack_cases(18, 20211120))
def test_random_stacks(et, H, nh, FF, S, B, nlayer, sp, mode, padded, causal, seed):
    """Seeded random encoder stacks through the model handle: hidden sizes 16 to 512, 1 to 8 heads of 16 to 64,
    1 to 3 layers, every precision mode (all binary16 storage, binary32 residual stream with SkipLayerNorm folded
    or launched), tile sparsities on both sides of the dense-image threshold, right padding, causal attention."""
    layers = [Hn.LayerWeights(H, nh, FF, sp, seed=seed + i) for i in range(nlayer)]
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, S + 1, B).astype(np.int32) if padded else None
    m = Hn.build_model(et, layers, S, B, lens=lens, causal=causal, mixed=mode)
    x = Hn.randn((B * S, H), seed ^ 0x77)
    got = run_model(et, m, x, reps=2)
    want = Hn.oracle_stack(x, layers, B, lens, causal=causal, store=torch.float16,
                           resid=torch.float32 if mode else "same")
    a, b = got[0].astype(np.float32), want.astype(np.float32)
    if lens is not None:  # rows past a sequence's length are padding: not compared
        for i in range(B):
            a[i * S + lens[i]:(i + 1) * S] = 0
            b[i * S + lens[i]:(i + 1) * S] = 0
    assert Hn.max_abs(a, b) <= (4e-3 if mode else TOL_F16)
    assert np.array_equal(got[0], got[1])


@pytest.mark.parametrize("mixed", [False, True])
def test_layer_at_4096_rows_uses_the_streaming_linear(et, mixed):
    """32 sequences of 128 tokens: the FFN down-projection (3072 inputs, 4096 token rows) runs on the
    planned streaming kernel inside the class layer; binary16 and binary32 results of it."""
    H, nh, FF, S, B = 768, 12, 3072, 128, 32
    layers = [Hn.LayerWeights(H, nh, FF, 0.8, seed=400)]
    m = Hn.build_model(et, layers, S, B, mixed=mixed)
    x = Hn.randn((B * S, H), 401)
    got = run_model(et, m, x, reps=2)
    want = Hn.oracle_stack(x, layers, B, store=torch.float16, resid=torch.float32 if mixed else "same")
    assert Hn.max_abs(got[0], want) <= 4e-3
    assert np.array_equal(got[0], got[1])


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_stack_of_weights_that_keep_most_tiles(et, mode):
    """20 % tile sparsity: the class multiplies with a dense image of each weight, and the
    mixed-precision engine keeps SkipLayerNorm as launches of its own (nothing to fold it into)."""
    H, nh, FF, S, B = 128, 2, 256, 32, 2
    layers = [Hn.LayerWeights(H, nh, FF, 0.2, seed=80 + i) for i in range(2)]
    m = Hn.build_model(et, layers, S, B, mixed=mode)
    x = Hn.randn((B * S, H), 96)
    got = run_model(et, m, x, reps=2)
    want = Hn.oracle_stack(x, layers, B, store=torch.float16, resid=torch.float32 if mode else "same")
    assert Hn.max_abs(got[0], want) <= (4e-3 if mode else TOL_F16)
    assert np.array_equal(got[0], got[1])


def test_in_place_forward_with_graph_all_fp16(et):
    H, nh, FF, S, B = 128, 2, 256, 32, 1
    layers = [Hn.LayerWeights(H, nh, FF, 0.5, seed=70 + i) for i in range(2)]
    m = Hn.build_model(et, layers, S, B)
    x = Hn.randn((B * S, H), 97)
    ref = run_model(et, m, x)[0]
    d = et.DeviceBuffer.from_numpy(x)
    m.forward(d, d)  # first call for this buffer pair: eager warm-up, capture, replay
    m.sync()
    assert np.array_equal(d.numpy(), ref)


def test_dense_single_layer_config(et):
    """Single BERT-base layer, dense weights N(0,0.02), biases 0, gamma 1 / beta 0, B1 S128."""
    H, nh, FF, S = 768, 12, 3072, 128
    g = Hn.rng(1)
    W = {k: (torch.randn(o, i, generator=g) * 0.02).numpy().astype(np.float16)
         for k, (o, i) in {"qkv": (3 * H, H), "o": (H, H), "l1": (FF, H), "l2": (H, FF)}.items()}
    m = et.Model(H, nh, FF, S, 1, batch=1, act=et.ACT_GELU)
    for which, k in ((et.W_QKV, "qkv"), (et.W_O, "o"), (et.W_FF1, "l1"), (et.W_FF2, "l2")):
        m.set_dense(0, which, W[k], None)
    ones, zeros = np.ones(H, np.float16), np.zeros(H, np.float16)
    m.set_norm(0, 0, ones, zeros)
    m.set_norm(0, 1, ones, zeros)
    m.finalize()
    x = Hn.randn((S, H), 6)
    got = run_model(et, m, x)[0]
    from oracle import layers as L
    P = L.LayerParams(Hn.f32(W["qkv"]), torch.zeros(3 * H), Hn.f32(W["o"]), torch.zeros(H), Hn.f32(W["l1"]),
                      torch.zeros(FF), Hn.f32(W["l2"]), torch.zeros(H), torch.ones(H), torch.zeros(H),
                      torch.ones(H), torch.zeros(H))
    want = L.encoder_layer(Hn.f32(x), P, L.LayerConfig(nh=nh, store=torch.float16)).numpy()
    assert Hn.max_abs(got, want) <= TOL_F16


def test_loader_from_npz_archives(et, tmp_path):
    """weights.txt + .npz archives written with numpy (np.savez, the exporter's writer) load into
    the same model as handing the arrays over directly."""
    H, nh, FF, S, B = 128, 2, 256, 32, 1
    layers = [Hn.LayerWeights(H, nh, FF, 0.5, seed=50 + i) for i in range(2)]
    names = []
    for i, w in enumerate(layers):
        pre = f"transformer_encoder.layers.{i}."
        for nm, bw in (("self_attn.in_proj_", w.qkv), ("self_attn.out_proj.", w.o), ("linear1.", w.l1),
                       ("linear2.", w.l2)):
            F.save_weight_npz(str(tmp_path / (pre + nm)), bw.dense.astype(np.float32), bw.bias.astype(np.float32))
            names.append(pre + nm + ".npz")
        for nm, (g, b) in (("norm1.", (w.g1, w.be1)), ("norm2.", (w.g2, w.be2))):
            F.save_weight_npz(str(tmp_path / (pre + nm)), g.astype(np.float32), b.astype(np.float32))
            names.append(pre + nm + ".npz")
    (tmp_path / "weights.txt").write_text("\n".join(names) + "\n")
    m = et.Model.load(tmp_path / "weights.txt", str(tmp_path) + "/", H, nh, FF, S, 2, batch=B)
    x = Hn.randn((S, H), 7)
    got = run_model(et, m, x)[0]
    direct = run_model(et, Hn.build_model(et, layers, S, B), x)[0]
    # the exporter drops all-zero tiles and sorts columns; values are identical, order of
    # accumulation inside a block-row may differ
    assert Hn.max_abs(got, direct) <= 4e-3
    assert Hn.max_abs(got, Hn.oracle_stack(x, layers, B)) <= TOL_F16


def test_model_rejects_bad_use(et, tmp_path):
    m = et.Model(128, 2, 256, 32, 1)
    with pytest.raises(et.EtError):
        m.finalize()  # nothing set
    with pytest.raises(et.EtError):
        m.set_bsr16(0, et.W_O, np.array([0, 1, 2, 3, 4, 5, 6, 7, 9], np.int32), np.zeros(8, np.int32),
                    np.zeros((8, 256), np.float16), None)  # row_ptr.back() != ntile
    with pytest.raises(et.EtError):
        m.set_norm(3, 0, np.ones(128, np.float16), np.ones(128, np.float16))  # layer out of range
    with pytest.raises(et.EtError):
        et.Model.load(tmp_path / "missing.txt", str(tmp_path) + "/", 128, 2, 256, 32, 1)
    with pytest.raises(et.EtError):
        et.Model(100, 3, 256, 32, 1)  # kdim % nhead != 0
