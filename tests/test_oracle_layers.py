"""The layer oracle pinned against PyTorch's own library routines and algebraic identities
(CPU only).  A dropped term, a wrong sign, a transposed operand or a wrong head slicing in
oracle/layers.py fails at least one of these."""
import math
from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle import formats as F
from oracle import layers as L

GOLDEN = Path(__file__).resolve().parent / "golden"


def g(seed):
    return torch.Generator().manual_seed(seed)


def test_gelu_tanh_matches_library():
    x = torch.linspace(-8, 8, 4001)
    assert torch.allclose(L.gelu_tanh(x), TF.gelu(x, approximate="tanh"), atol=2e-7)
    assert L.gelu_tanh(torch.tensor(0.0)) == 0 and abs(L.gelu_tanh(torch.tensor(1.0)).item() - 0.8411920) < 1e-6
    # the tanh form is NOT the erf form: they differ by more than the fp32 tolerance of the engine
    assert (L.gelu_tanh(x) - TF.gelu(x)).abs().max() > 1e-4


def test_layernorm_matches_library_and_invariants():
    x = torch.randn(37, 768, generator=g(1)) * 3 + 1
    skip = torch.randn(37, 768, generator=g(2))
    gamma, beta = torch.randn(768, generator=g(3)), torch.randn(768, generator=g(4))
    want = TF.layer_norm(x + skip, (768,), gamma, beta, 1e-5)
    assert torch.allclose(L.skip_layernorm(x, skip, gamma, beta, 1e-5), want, atol=2e-5)
    assert torch.allclose(L.layernorm(x, gamma, beta, 1e-5), TF.layer_norm(x, (768,), gamma, beta, 1e-5), atol=2e-5)
    y = L.skip_layernorm(x, skip, torch.ones(768), torch.zeros(768), 1e-5)
    assert y.mean(-1).abs().max() < 1e-5 and (y.var(-1, unbiased=False) - 1).abs().max() < 1e-3
    # the reference's flawed variance (E[x^2] - mean, SkipLayerNorm.cu:50-52) would not pass:
    bad = ((x + skip) - (x + skip).mean(-1, keepdim=True)) / torch.sqrt(((x + skip) ** 2).mean(-1, keepdim=True) - (x + skip).mean(-1, keepdim=True) + 1e-5)
    assert not torch.allclose(bad * gamma + beta, want, atol=1e-2)


def test_linear_orientation_and_pruned_forms():
    x = torch.randn(20, 48, generator=g(5))
    W = torch.randn(32, 48, generator=g(6))
    b = torch.randn(32, generator=g(7))
    assert torch.allclose(L.linear(x, W, b), TF.linear(x, W, b), atol=1e-5)
    assert torch.allclose(L.linear(x, W, b, "relu"), TF.relu(TF.linear(x, W, b)), atol=1e-5)
    # row-pruned: pruned output features carry the bias alone
    row_id = np.array([1, 4, 5, 30])
    y = L.linear_rowpruned(x, W[row_id], row_id, 32, b)
    Wm = torch.zeros_like(W); Wm[row_id] = W[row_id]
    assert torch.allclose(y, TF.linear(x, Wm, b), atol=1e-5)
    assert torch.allclose(y[:, 0], b[0].expand(20))
    # column-pruned with unsorted ids
    col_id = np.array([40, 2, 17, 3])
    Wc = torch.zeros_like(W); Wc[:, col_id] = W[:, col_id]
    assert torch.allclose(L.linear_colpruned(x, W[:, col_id], col_id, b), TF.linear(x, Wc, b), atol=1e-5)
    # BSR weights as masked dense matrices: round trip through the format oracle
    Wd = torch.randn(64, 96, generator=g(8)).numpy() * np.kron(np.random.default_rng(0).random((4, 6)) < 0.5, np.ones((16, 16)))
    rp, col, data = F.dense_to_bsr16(Wd.astype(np.float32))
    assert np.array_equal(F.bsr16_to_dense(rp, col, data, 96), Wd.astype(np.float32))


@pytest.mark.parametrize("B,S,nh,hd", [(1, 128, 12, 64), (3, 32, 4, 16)])
def test_mha_matches_sdpa(B, S, nh, hd):
    H = nh * hd
    q, k, v = (torch.randn(B * S, H, generator=g(10 + i)) for i in range(3))
    split = lambda t: t.reshape(B, S, nh, hd).permute(0, 2, 1, 3)
    merge = lambda t: t.permute(0, 2, 1, 3).reshape(B * S, H)
    want = merge(TF.scaled_dot_product_attention(split(q), split(k), split(v)))
    assert torch.allclose(L.mha(q, k, v, nh, B), want, atol=2e-5)
    # causal
    want_c = merge(TF.scaled_dot_product_attention(split(q), split(k), split(v), is_causal=True))
    assert torch.allclose(L.mha(q, k, v, nh, B, causal=True), want_c, atol=2e-5)
    assert torch.allclose(L.mha(q, k, v, nh, B, mask=L.additive_mask(S, "causal")), want_c, atol=2e-5)
    # additive mask + right padding as one boolean/additive mask for the library
    lens = torch.tensor([S, S // 2, S - 3][:B])
    add = torch.randn(S, S, generator=g(20))
    full = add[None, None].expand(B, 1, S, S).clone()
    for b in range(B):
        full[b, :, :, int(lens[b]):] = float("-inf")
    want_m = merge(TF.scaled_dot_product_attention(split(q), split(k), split(v), attn_mask=full))
    z, P = L.mha(q, k, v, nh, B, mask=add, lens=lens, return_probs=True)
    assert torch.allclose(z, want_m, atol=2e-5)
    # invariants: rows of P sum to one, padded keys weigh exactly zero
    assert torch.allclose(P.sum(-1), torch.ones(B, nh, S), atol=1e-5)
    for b in range(B):
        assert torch.all(P[b, :, :, int(lens[b]):] == 0)
    # a custom scale is honoured
    want_s = merge(TF.scaled_dot_product_attention(split(q), split(k), split(v), scale=0.3))
    assert torch.allclose(L.mha(q, k, v, nh, B, scale=0.3), want_s, atol=2e-5)


def test_mha_head_permutation_and_batch_independence():
    B, S, nh, hd = 2, 16, 4, 8
    H = nh * hd
    q, k, v = (torch.randn(B * S, H, generator=g(30 + i)) for i in range(3))
    z = L.mha(q, k, v, nh, B)
    perm = [2, 0, 3, 1]
    cols = torch.cat([torch.arange(h * hd, (h + 1) * hd) for h in perm])
    assert torch.allclose(L.mha(q[:, cols], k[:, cols], v[:, cols], nh, B), z[:, cols], atol=1e-6)
    assert torch.allclose(L.mha(q[S:], k[S:], v[S:], nh, 1), z[S:], atol=1e-6)


def test_encoder_layer_matches_torch_transformer_layer_fixture():
    """oracle.layers.encoder_layer == torch.nn.TransformerEncoderLayer (post-norm, tanh GELU,
    eps 1e-5) on the dense BERT-base configuration; the library output is a committed fixture
    (tests/golden/make_encoder_layer_c1.py)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("mk", GOLDEN / "make_encoder_layer_c1.py")
    mk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mk)
    p = mk.seeded_params()
    H, FF = mk.H, mk.FF
    P = L.LayerParams(p["Wqkv"], torch.zeros(3 * H), p["Wo"], torch.zeros(H), p["W1"], torch.zeros(FF), p["W2"],
                      torch.zeros(H), torch.ones(H), torch.zeros(H), torch.ones(H), torch.zeros(H))
    y = L.encoder_layer(p["x"], P, L.LayerConfig(nh=mk.NH, act="gelu", eps=1e-5))
    fx = np.load(GOLDEN / "encoder_layer_c1.npz")
    assert np.max(np.abs(y[:8].numpy() - fx["y_head"])) <= 1e-4  # the fp32-path tolerance
    assert abs(y.double().sum().item() - float(fx["y_sum"])) <= 1e-2
    assert abs(y.double().abs().sum().item() - float(fx["y_abs_sum"])) <= 1e-1 


def test_encoder_layer_live_against_torch_layer_with_biases_relu_and_padding():
    H, nh, FF, S, B = 64, 4, 128, 16, 2
    layer = torch.nn.TransformerEncoderLayer(H, nh, FF, dropout=0.0, activation="relu", layer_norm_eps=1e-5,
                                             batch_first=True, norm_first=False).eval()
    torch.manual_seed(3)
    with torch.no_grad():
        for prm in layer.parameters():
            prm.copy_(torch.randn_like(prm) * 0.2)
    sd = layer.state_dict()
    P = L.LayerParams(sd["self_attn.in_proj_weight"], sd["self_attn.in_proj_bias"], sd["self_attn.out_proj.weight"],
                      sd["self_attn.out_proj.bias"], sd["linear1.weight"], sd["linear1.bias"], sd["linear2.weight"],
                      sd["linear2.bias"], sd["norm1.weight"], sd["norm1.bias"], sd["norm2.weight"], sd["norm2.bias"])
    x = torch.randn(B, S, H)
    lens = torch.tensor([16, 9])
    pad = torch.arange(S)[None, :] >= lens[:, None]
    with torch.no_grad():
        want = layer(x, src_key_padding_mask=pad)
    got = L.encoder_layer(x.reshape(B * S, H), P, L.LayerConfig(nh=nh, B=B, act="relu", lens=lens)).reshape(B, S, H)
    for b in range(B):  # torch zeroes/ignores padded query rows on its fast path; compare the valid ones
        n = int(lens[b])
        assert torch.allclose(got[b, :n], want[b, :n], atol=2e-5)


def test_fused_vo_identity():
    """sum_h P_h (X W_VO,h + b_VO,h) + b_O equals standard attention + output projection when
    W_VO,h = W_V,h^T W_O[:, h]^T and b_VO,h = b_V,h W_O[:, h]^T."""
    H, nh, S, B = 64, 4, 16, 2
    hd = H // nh
    gg = g(40)
    rn = lambda *s: torch.randn(*s, generator=gg) * 0.3
    x = rn(B * S, H)
    Wq, Wk, Wv, Wo = rn(H, H), rn(H, H), rn(H, H), rn(H, H)
    bq, bk, bv, bo = rn(H), rn(H), rn(H), rn(H)
    Wvo = torch.stack([Wv[h * hd:(h + 1) * hd].T @ Wo[:, h * hd:(h + 1) * hd].T for h in range(nh)])
    bvo = torch.stack([bv[h * hd:(h + 1) * hd] @ Wo[:, h * hd:(h + 1) * hd].T for h in range(nh)])
    lens = torch.tensor([16, 11])
    fused = L.fused_vo_attention(x, x, x, Wq, bq, Wk, bk, Wvo, bvo, bo, nh, B, lens=lens)
    z = L.mha(L.linear(x, Wq, bq), L.linear(x, Wk, bk), L.linear(x, Wv, bv), nh, B, lens=lens)
    assert torch.allclose(fused, L.linear(z, Wo, bo), atol=2e-5)


def test_fp16_storage_oracle_stays_within_the_fp16_tolerance_of_the_fp32_math():
    """Rounding at the engine's storage points moves a layer output by far less than 2e-2."""
    H, nh, FF, S = 128, 4, 256, 32
    gg = g(50)
    rn = lambda *s: (torch.randn(*s, generator=gg) * 0.05).half().float()
    P = L.LayerParams(rn(3 * H, H), rn(3 * H), rn(H, H), rn(H), rn(FF, H), rn(FF), rn(H, FF), rn(H),
                      torch.ones(H), torch.zeros(H), torch.ones(H), torch.zeros(H))
    x = torch.randn(S, H, generator=gg).half().float()
    y32 = L.encoder_layer(x, P, L.LayerConfig(nh=nh))
    y16 = L.encoder_layer(x, P, L.LayerConfig(nh=nh, store=torch.float16))
    assert (y32 - y16).abs().max() < 1e-2
    assert (y32 - y16).abs().max() > 0  # the rounding is really applied
