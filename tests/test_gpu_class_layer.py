"""The C++ class layer used directly, as a caller written against the reference's headers would
(tests/cpp/class_layer_cases.cpp): example-style model assembly from weights.txt + .npz, the
attention-aware Prune_attn form, FusedAttention (dense and column-pruned W_VO) and the gen_*
factories.  The program writes .npy files; the CPU oracle is the judge."""
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import layers as L
from tests import harness as Hn

pytestmark = pytest.mark.gpu

EXE = Path(__file__).resolve().parent / "cpp" / "bin" / "class_layer_cases"


def run_case(case, d):
    assert EXE.exists(), f"{EXE} is missing: build it with `python scpaper-2021_amd/build.py`"
    res = subprocess.run([str(EXE), case, str(d)], capture_output=True, text=True, timeout=120)
    print(res.stdout, res.stderr)
    assert res.returncode == 0, res.stderr
    return res


def write_example_model(tmp_path, layers, dec, x, S, B):
    """weights.txt + one .npz per weight in the reference example's naming (example/main.cu:40-160)."""
    H, nh, FF = layers[0].H, layers[0].nh, layers[0].dimFF
    names = []
    for i, w in enumerate(layers):
        pre = f"transformer_encoder.layers.{i}."
        for nm, bw in (("self_attn.in_proj_", w.qkv), ("self_attn.out_proj.", w.o), ("linear1.", w.l1), ("linear2.", w.l2)):
            F.save_weight_npz(str(tmp_path / (pre + nm)), bw.dense.astype(np.float32), bw.bias.astype(np.float32))
            names.append(pre + nm + ".npz")
        for nm, (g, b) in (("norm1.", (w.g1, w.be1)), ("norm2.", (w.g2, w.be2))):
            F.save_weight_npz(str(tmp_path / (pre + nm)), g.astype(np.float32), b.astype(np.float32))
            names.append(pre + nm + ".npz")
    F.save_weight_npz(str(tmp_path / "decoder."), dec.dense.astype(np.float32), dec.bias.astype(np.float32))
    names.append("decoder..npz")
    (tmp_path / "weights.txt").write_text("\n".join(names) + "\n")
    np.save(tmp_path / "input.npy", x.astype(np.float32))
    np.save(tmp_path / "meta.npy", np.array([H, H, S, nh, FF, H, len(layers), B, dec.out], np.int32))


@pytest.mark.parametrize("H,S,TEXT", [(512, 64, 1024), (512, 64, 28800), (800, 128, 28800)])
def test_example_model_from_npz(tmp_path, H, S, TEXT):
    """Two ReLU encoder layers + decoder assembled as the reference example does.  H 800, 4 heads x 200,
    FFN 208, seq 128, decoder 28 800 wide is the example's own Model_t{800, 800, 128, 4, 208, 800, 2}
    (example/main.cu:24-31,164); H 512, 4 heads x 128 is a smaller member of the family."""
    nh, FF, B, NL = 4, 208, 2, 2
    layers = [Hn.LayerWeights(H, nh, FF, 0.6, seed=70 + i) for i in range(NL)]
    dec = Hn.BsrWeight(TEXT, H, 0.7, seed=90, bias_std=0.02)
    x = Hn.randn((B * S, H), 91)
    write_example_model(tmp_path, layers, dec, x, S, B)
    res = run_case("example", tmp_path)
    assert "encoder layer forward" in res.stdout
    hidden = Hn.oracle_stack(x, layers, B, act="relu")
    want = L.linear(torch.from_numpy(hidden), Hn.f32(dec.dense), Hn.f32(dec.bias), None, torch.float16).numpy()
    assert Hn.max_abs(np.load(tmp_path / "hidden.npy"), hidden) <= 2e-2
    assert Hn.max_abs(np.load(tmp_path / "out.npy"), want) <= 2e-2


def test_twelve_class_layers_through_forward(tmp_path):
    """Twelve BERT-base Encoder<> objects (80 % tile sparsity, ReLU) called one after the other through the
    reference's own signature, forward(half *out, half *src), as example/main.cu:175-177 does: the result of
    layer 12 stays within the 2e-2 asked of the fp16 path, measured against the fp32 mathematics, because the
    residual stream is binary32 inside each layer and binary16 only between layers.  Measured 9.7e-3, and the
    CPU oracle rounding at the same places is 9.7e-3 from the fp32 mathematics too: values reach 7.8, where one
    binary16 step is 7.8e-3, and every layer boundary rounds once.  (All-binary16 storage: 1.6e-2 on these
    weights, 2.3e-2 .. 5e-2 on the GELU headline stack.)"""
    H, nh, FF, S, B, NL, TEXT = 768, 12, 3072, 128, 2, 12, 256
    layers = [Hn.LayerWeights(H, nh, FF, 0.8, seed=700 + i) for i in range(NL)]
    dec = Hn.BsrWeight(TEXT, H, 0.8, seed=790, bias_std=0.02)
    x = Hn.randn((B * S, H), 791)
    write_example_model(tmp_path, layers, dec, x, S, B)
    run_case("example", tmp_path)
    got = np.load(tmp_path / "hidden.npy")
    want32 = Hn.oracle_stack(x, layers, B, act="relu", store=None)
    want = Hn.oracle_stack(x, layers, B, act="relu", store=torch.float16, resid=torch.float32, boundary=torch.float16)
    e32, eo = Hn.max_abs(got, want32), Hn.max_abs(got, want)
    print(f"12 class layers through forward(): vs fp32 forward {e32:.3e}, vs the oracle rounding where the classes do {eo:.3e}")
    assert e32 <= 2e-2 and eo <= 1.6e-2  # the asked bound; two binary16 steps at |x| < 8 between two realisations


def attention_inputs(tmp_path, H, nh, S, B, seed):
    g = Hn.rng(seed)
    rn = lambda *s: (torch.randn(*s, generator=g) * 0.05).numpy().astype(np.float16)
    W = {k: rn(H, H) for k in "qkvo"}
    b = {k: rn(H) for k in "qkvo"}
    x = Hn.randn((B * S, H), seed + 1)
    lens = np.array([S, S - 11][:B], np.int32)
    for k in "qkvo":
        np.save(tmp_path / f"W{k}.npy", W[k].astype(np.float32))
        np.save(tmp_path / f"b{k}.npy", b[k].astype(np.float32))
    np.save(tmp_path / "input.npy", x.astype(np.float32))
    np.save(tmp_path / "lens.npy", lens)
    np.save(tmp_path / "meta.npy", np.array([H, S, nh, B], np.int32))
    return W, b, x, lens


def test_prune_attn_class(tmp_path):
    """Attention<tile, tile, row_mat, tile, Prune_attn>: W_V row-pruned, V kept compact, P*V over
    the surviving columns, Z full width — equals standard attention with the pruned W_V rows (and
    their bias) zero."""
    H, nh, S, B = 256, 4, 64, 2
    W, b, x, lens = attention_inputs(tmp_path, H, nh, S, B, 110)
    row_id = F.gen_row_ids(H, 0.25, seed=5)  # 192 of 256 V features survive
    np.save(tmp_path / "v_row_id.npy", row_id)
    np.save(tmp_path / "v_rows.npy", W["v"][row_id].astype(np.float32))
    run_case("prune_attn", tmp_path)
    Wv = np.zeros_like(W["v"]); Wv[row_id] = W["v"][row_id]
    bv = np.zeros_like(b["v"]); bv[row_id] = b["v"][row_id]
    st = torch.float16
    q = L.linear(Hn.f32(x), Hn.f32(W["q"]), Hn.f32(b["q"]), store=st)
    k = L.linear(Hn.f32(x), Hn.f32(W["k"]), Hn.f32(b["k"]), store=st)
    v = L.linear(Hn.f32(x), Hn.f32(Wv), Hn.f32(bv), store=st)
    z = L.mha(q, k, v, nh, B, lens=lens, store=st)
    want = L.linear(z, Hn.f32(W["o"]), Hn.f32(b["o"]), store=st).numpy()
    assert Hn.max_abs(np.load(tmp_path / "out.npy"), want) <= 6e-3


@pytest.mark.parametrize("case", ["fused_attn", "fused_otf", "fused_prune"])
def test_fused_attention_class(tmp_path, case):
    """FusedAttention with W_VO built by et::build_vo_weight equals standard attention followed by
    the output projection (the E.T. identity); the pruned form keeps half of the W_VO columns."""
    H, nh, S, B = 256, 4, 64, 2
    W, b, x, lens = attention_inputs(tmp_path, H, nh, S, B, 120)
    hd = H // nh
    col_id = np.sort(F.gen_col_ids(H, 0.5, seed=6)).astype(np.int32)
    np.save(tmp_path / "vo_col_id.npy", col_id)
    run_case(case, tmp_path)
    f = lambda a: a.astype(np.float32)
    Wvo = np.stack([f(W["v"])[h * hd:(h + 1) * hd].T @ f(W["o"])[:, h * hd:(h + 1) * hd].T for h in range(nh)])
    bvo = np.stack([f(b["v"])[h * hd:(h + 1) * hd] @ f(W["o"])[:, h * hd:(h + 1) * hd].T for h in range(nh)])
    assert Hn.max_abs(np.load(tmp_path / "Wvo.npy"), Wvo) <= 1e-5  # the offline builder
    assert Hn.max_abs(np.load(tmp_path / "bvo.npy"), bvo) <= 1e-5
    st = torch.float16
    if case == "fused_prune":
        m = np.zeros(H, bool); m[col_id] = True
        Wvo, bvo = Wvo * m, bvo * m
    Wvo16, bvo16 = torch.from_numpy(Wvo).half().float(), torch.from_numpy(bvo).half().float()
    want = L.fused_vo_attention(Hn.f32(x), Hn.f32(x), Hn.f32(x), Hn.f32(W["q"]), Hn.f32(b["q"]), Hn.f32(W["k"]),
                                Hn.f32(b["k"]), Wvo16, bvo16, Hn.f32(b["o"]), nh, B, lens=lens, store=st).numpy()
    got = np.load(tmp_path / "out.npy")
    assert Hn.max_abs(got, want) <= 6e-3
    if case in ("fused_attn", "fused_otf"):  # and the identity with plain attention + output projection
        q = L.linear(Hn.f32(x), Hn.f32(W["q"]), Hn.f32(b["q"]), store=st)
        k = L.linear(Hn.f32(x), Hn.f32(W["k"]), Hn.f32(b["k"]), store=st)
        v = L.linear(Hn.f32(x), Hn.f32(W["v"]), Hn.f32(b["v"]))
        std = L.linear(L.mha(q, k, v, nh, B, lens=lens), Hn.f32(W["o"]), Hn.f32(b["o"])).numpy()
        assert Hn.max_abs(got, std) <= 2e-2


def test_factories_closed_forms(tmp_path):
    run_case("factories", tmp_path)
    v = np.load(tmp_path / "factories.npy").tolist()
    dense_b, dense_t, sp_got, sp_want, sp_ntile, row_dense, row_live, row_dead, row_n, col_v, csr_v, v16, vo, ln, *db = v
    assert dense_b == 256.5 and dense_t == 256.5
    assert sp_got == sp_want and sp_ntile == 64
    assert row_dense == 256.5 and row_live == 256.5 and row_dead == 0.5 and row_n == 64
    assert col_v == 64.5 and csr_v == 256.5 and v16 == 256.5
    assert vo == 205.0  # the reference driver's expected value (Fused_attention/test/testVO.cu:10-16)
    assert abs(ln - 0.2) < 1e-3
    # Linear<csr_mat>: dense-image path (80 %) and CSR-kernel path (99 %) both equal the CSR kernel called directly
    assert db[:4] == [1.0, 1.0, 1.0, 0.0]
    assert db[4:8] == [3.0, 4.0, 0.0, 1.0]
    assert db[8:10] == [7.0, 6.0]  # DeviceBuffer(ptr, n) from a device pointer and from a host pointer
    assert db[10] == db[11] and db[10] > 32.0  # Linear<tile_mat>::refresh() after the caller rewrote weight.data
    # Linear<row_mat>, 512 features: half kept -> dense image; 1 in 16 kept -> fill + scattering GEMM
    assert db[12:17] == [256.5, 0.5, 256.5, 256.0, 1.0]
    assert db[17:22] == [256.5, 0.5, 256.5, 32.0, 0.0]


def test_attention_tags_with_separate_projections(tmp_path):
    """Attention<> with separate Q/K/V projections under OTF_attn_full, OTF_attn_full_mixed, OTF_attn,
    OTF_attn_Ofused (tile-sparse weights) and Norm_attn (dense weights, scores through memory), the
    binary32-output form, and the free Multihead_atttion_fuseO: all the standard attention block."""
    H, nh, S, B = 256, 4, 64, 2
    W, b, x, lens = attention_inputs(tmp_path, H, nh, S, B, 130)
    run_case("attn_variants", tmp_path)
    st = torch.float16
    lin = lambda t, inp, store=st: L.linear(inp, Hn.f32(W[t]), Hn.f32(b[t]), store=store)
    xf = Hn.f32(x)
    z = L.mha(lin("q", xf), lin("k", xf), lin("v", xf), nh, B, lens=lens, store=st)
    want = lin("o", z).numpy()
    full = np.load(tmp_path / "out_full.npy")
    assert Hn.max_abs(full, want) <= 4e-3
    for name in ("out_full_mixed.npy", "out_ofused.npy", "out_otf.npy"):
        assert np.array_equal(np.load(tmp_path / name), full), name  # one fused kernel behind every on-the-fly tag
    assert Hn.max_abs(np.load(tmp_path / "out_norm.npy"), want) <= 6e-3  # probabilities rounded to fp16 in memory
    want32 = lin("o", z, None).numpy()
    assert Hn.max_abs(np.load(tmp_path / "out_full_f32.npy"), want32) <= 1e-3
    assert np.array_equal(np.load(tmp_path / "out_full_f32.npy").astype(np.float16), full.astype(np.float16))
    assert Hn.max_abs(np.load(tmp_path / "out_dense_f32.npy"), want) <= 4e-3
    # free function: attention over Q = K = V = x without projections, no padding, then the O projection
    z0 = L.mha(xf, xf, xf, nh, B, store=st)
    assert Hn.max_abs(np.load(tmp_path / "out_fuseO_free.npy"), lin("o", z0).numpy()) <= 6e-3
    assert Hn.max_abs(np.load(tmp_path / "out_fuseO_one_launch.npy"), lin("o", z0).numpy()) <= 6e-3


def test_encoder_fuse_class(tmp_path):
    """Encoder_fuse: pre-computed-VO attention, SkipLayerNorm, tile-sparse FFN with GELU — equals the
    standard layer (the E.T. identity); and the same layer with a binary32 residual stream."""
    H, nh, S, B, FF = 256, 4, 64, 2, 512
    W, b, x, lens = attention_inputs(tmp_path, H, nh, S, B, 140)
    w1 = Hn.BsrWeight(FF, H, 0.5, seed=141, bias_std=0.02)
    w2 = Hn.BsrWeight(H, FF, 0.5, seed=142, bias_std=0.02)
    g = {k: (1 + Hn.randn((H,), 143 + i, 0.1, np.float32)).astype(np.float16) for i, k in enumerate("12")}
    be = {k: Hn.randn((H,), 146 + i, 0.1) for i, k in enumerate("12")}
    for k in "12":
        np.save(tmp_path / f"g{k}.npy", g[k].astype(np.float32))
        np.save(tmp_path / f"be{k}.npy", be[k].astype(np.float32))
    np.save(tmp_path / "W1.npy", w1.dense.astype(np.float32)); np.save(tmp_path / "b1.npy", w1.bias.astype(np.float32))
    np.save(tmp_path / "W2.npy", w2.dense.astype(np.float32)); np.save(tmp_path / "b2.npy", w2.bias.astype(np.float32))
    np.save(tmp_path / "meta.npy", np.array([H, S, nh, B, FF], np.int32))
    run_case("encoder_fuse", tmp_path)
    Wqkv = np.concatenate([W["q"], W["k"], W["v"]]); bqkv = np.concatenate([b["q"], b["k"], b["v"]])
    P = L.LayerParams(Hn.f32(Wqkv), Hn.f32(bqkv), Hn.f32(W["o"]), Hn.f32(b["o"]), Hn.f32(w1.dense), Hn.f32(w1.bias),
                      Hn.f32(w2.dense), Hn.f32(w2.bias), Hn.f32(g["1"]), Hn.f32(be["1"]), Hn.f32(g["2"]), Hn.f32(be["2"]))
    cfg = lambda **kw: L.LayerConfig(nh=nh, B=B, act="gelu", lens=torch.as_tensor(lens), **kw)
    want32 = L.encoder_layer(Hn.f32(x), P, cfg(store=None)).numpy()
    # the VO form rounds different intermediates than the standard layer: both within the layer tolerance
    assert Hn.max_abs(np.load(tmp_path / "out.npy"), want32) <= 2e-2
    m32, m16 = np.load(tmp_path / "out_mixed32.npy"), np.load(tmp_path / "out_mixed16.npy")
    assert Hn.max_abs(m32, want32) <= 1e-2
    assert np.array_equal(m16.astype(np.float16), m32.astype(np.float16))
    # forward(half*, half*) keeps the residual stream binary32 inside the layer: the mixed form's binary16 result
    assert np.array_equal(np.load(tmp_path / "out_forward.npy"), m16)


def test_raw_file_constructors(tmp_path):
    """row_mat(std::string), col_mat(std::string), csr_mat(std::string) on hand-written byte strings
    (tests/golden/pruned_files.json) and on files whose header does not describe them."""
    import json
    g = json.loads((Path(__file__).resolve().parent / "golden" / "pruned_files.json").read_text())
    raw = {k: bytes.fromhex(g[k]["hex"].replace(" ", "")) for k in ("row", "col", "csr")}
    for k in raw:
        (tmp_path / f"small.{k}").write_bytes(raw[k])
        bad = bytearray(raw[k]); bad[8:12] = (100000).to_bytes(4, "little")  # len_id / nnz far beyond the file
        (tmp_path / f"bad.{k}").write_bytes(bytes(bad))
    run_case("file_ctors", tmp_path)
    ld = lambda n: np.load(tmp_path / n)
    r, c, s = g["row"], g["col"], g["csr"]
    assert ld("row_meta.npy").tolist() == [r["nrow"], r["ncol"], 2] and ld("row_id.npy").tolist() == r["row_id"]
    assert ld("rows.npy").tolist() == np.array(r["rows"]).ravel().tolist()
    assert ld("col_meta.npy").tolist() == [c["nrow"], c["ncol"], 2, 2] and ld("col_id.npy").tolist() == c["col_id"]
    assert ld("cols.npy").tolist() == np.array(c["cols"]).ravel().tolist()
    assert ld("csr_meta.npy").tolist() == [2, 3, 3] and ld("csr_indptr.npy").tolist() == s["indptr"]
    assert ld("csr_indices.npy").tolist() == s["indices"] and ld("csr_data.npy").tolist() == s["data"]
    assert ld("refused.npy").tolist() == [3]
