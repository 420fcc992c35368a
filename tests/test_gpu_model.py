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


def test_bert_base_12_layers_batch8_tile80_attention_aware(et):
    """The headline configuration: 12 layers, B8 S128, 80 % tile sparsity, 25 % of the V rows
    (and the matching O columns) dead in head-aligned 16-row groups."""
    H, nh, FF, S, B = 768, 12, 3072, 128, 8
    layers = [Hn.LayerWeights(H, nh, FF, 0.8, seed=100 + i, attention_aware=0.25) for i in range(12)]
    assert len(layers[0].qkv.col_idx) == F.tile_count(3 * H, H, 0.8)
    m = Hn.build_model(et, layers, S, B)
    x = Hn.randn((B * S, H), 4)
    got = run_model(et, m, x, reps=2)
    want = Hn.oracle_stack(x, layers, B)
    err = Hn.max_abs(got[0], want)
    print(f"12-layer B8 S128 max-abs={err:.3e}")
    assert err <= TOL_F16
    assert np.array_equal(got[0], got[1])


def test_bert_large_shape_padded_4_layers(et):
    """BERT-large shaped layers (H1024, 16 heads, FFN 4096, S512, B4, 90 % tiles, lengths in
    [256,512]); 4 of the 24 layers keep the CPU oracle within seconds."""
    H, nh, FF, S, B = 1024, 16, 4096, 512, 4
    layers = [Hn.LayerWeights(H, nh, FF, 0.9, seed=200 + i) for i in range(4)]
    lens = torch.randint(256, 513, (B,), generator=Hn.rng(5)).numpy().astype(np.int32)
    m = Hn.build_model(et, layers, S, B, lens=lens)
    x = Hn.randn((B * S, H), 5)
    got = run_model(et, m, x)[0]
    err = Hn.max_abs(got, Hn.oracle_stack(x, layers, B, lens))
    print(f"BERT-large shape lens={lens.tolist()} max-abs={err:.3e}")
    assert err <= TOL_F16


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
