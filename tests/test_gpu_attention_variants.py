"""GPU parity of the attention forms whose operands differ from the plain fused kernel:
probabilities in memory, the unfused baseline, the pre-computed-VO attention (dense and
column-pruned) and the attention-aware compact-V form."""
import math

import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import layers as L
from tests import harness as Hn

pytestmark = pytest.mark.gpu


up = Hn.up


@pytest.mark.parametrize("B,S,nh,hd,causal", [(2, 128, 12, 64, False), (1, 512, 4, 64, True), (3, 48, 2, 32, False)])
def test_probs_and_unfused(et, B, S, nh, hd, causal):
    H, T = nh * hd, B * S
    q, k, v = Hn.randn((T, H), 1), Hn.randn((T, H), 2), Hn.randn((T, H), 3)
    lens = np.array([S, S // 2 + 1, S - 5][:B], np.int32)
    d_p = et.DeviceBuffer.empty((T, nh * S), np.float16)
    d_z = et.DeviceBuffer.empty((T, H), np.float16)
    flags = et.MHA_CAUSAL if causal else 0
    scale = 1 / math.sqrt(hd)
    et.check(et.lib().et_mha_unfused_f16(up(et, q).ptr, up(et, k).ptr, up(et, v).ptr, H, H, H, d_z.ptr, H, d_p.ptr, None,
                                         up(et, lens).ptr, B, S, nh, hd, scale, flags, None))
    z, P = L.mha(Hn.f32(q), Hn.f32(k), Hn.f32(v), nh, B, lens=lens, causal=causal, return_probs=True)
    got_p = d_p.numpy().astype(np.float32).reshape(B, S, nh, S).transpose(0, 2, 1, 3)  # [b][h][q][key]
    assert Hn.max_abs(got_p, P.numpy()) <= 1e-3
    assert abs(got_p.sum(-1) - 1).max() <= 4e-3
    for b in range(B):
        assert np.all(got_p[b, :, :, lens[b]:] == 0)
    assert Hn.max_abs(d_z.numpy(), z.numpy()) <= 4e-3


def vo_case(seed, H, nh, N_keep=None):
    g = Hn.rng(seed)
    rn = lambda *s: (torch.randn(*s, generator=g) * 0.05)
    Wq, Wk, Wv, Wo = rn(H, H), rn(H, H), rn(H, H), rn(H, H)
    bq, bk, bv, bo = rn(H), rn(H), rn(H), rn(H)
    hd = H // nh
    Wvo = torch.stack([Wv[h * hd:(h + 1) * hd].T @ Wo[:, h * hd:(h + 1) * hd].T for h in range(nh)])  # [nh][H][H]
    bvo = torch.stack([bv[h * hd:(h + 1) * hd] @ Wo[:, h * hd:(h + 1) * hd].T for h in range(nh)])
    h16 = lambda t: t.numpy().astype(np.float16)
    return dict(Wq=h16(Wq), Wk=h16(Wk), bq=h16(bq), bk=h16(bk), Wvo=h16(Wvo), bvo=h16(bvo), bo=h16(bo))


@pytest.mark.parametrize("B,S,H,nh,pruned", [(1, 128, 768, 12, False), (2, 64, 256, 4, False), (2, 64, 256, 4, True),
                                             (9, 48, 96, 3, True), (2, 272, 256, 2, False), (1, 128, 512, 8, False),
                                             (8, 128, 768, 12, False), (2, 64, 96, 2, False), (1, 32, 64, 4, True),
                                             (2, 96, 288, 3, True)])
def test_vo_attention(et, B, S, H, nh, pruned):
    """Linear_VO + probabilities + one GEMM per sequence == the oracle's sum_h P_h VO_h + b_O, and so
    does the kernel that keeps the probabilities on chip."""
    T, hd = B * S, H // nh
    c = vo_case(7, H, nh)
    x = Hn.randn((T, H), 8)
    lens = np.array([S, S - 9, 1, 0, S // 2, S, 17, S - 1, 5][:B], np.int32)
    Wvo, bvo = c["Wvo"], c["bvo"]
    col_id = None
    if pruned:
        col_id = np.sort(F.gen_col_ids(H, 0.5, seed=9)).astype(np.int32)
        Wvo, bvo = np.ascontiguousarray(Wvo[:, :, col_id]), np.ascontiguousarray(bvo[:, col_id])
    N = Wvo.shape[2]
    # Q, K projections through the dense Linear kernel
    d_q, d_k = et.DeviceBuffer.empty((T, H), np.float16), et.DeviceBuffer.empty((T, H), np.float16)
    d_x = up(et, x)
    et.linear_dense(up(et, c["Wq"]), up(et, c["bq"]), d_x, d_q, T, H, H)
    et.linear_dense(up(et, c["Wk"]), up(et, c["bk"]), d_x, d_k, T, H, H)
    d_vo = et.DeviceBuffer.empty((B, nh, S, N), np.float16)
    et.check(et.lib().et_linear_vo_f16(up(et, Wvo).ptr, up(et, bvo).ptr, d_x.ptr, d_vo.ptr, B, S, H, N, nh, None))
    want_vo = (x.astype(np.float32).reshape(B, 1, S, H) @ Wvo.astype(np.float32)[None] +
               bvo.astype(np.float32)[None, :, None, :]).astype(np.float16)
    assert Hn.max_abs(d_vo.numpy(), want_vo) <= 4e-3
    # the same projection from weights transposed per head on the device (what the classes use)
    d_wt = et.DeviceBuffer.empty((nh, N, H), np.float16)
    et.check(et.lib().et_transpose_heads_f16(d_wt.ptr, up(et, Wvo).ptr, nh, H, N, None))
    assert np.array_equal(d_wt.numpy(), np.ascontiguousarray(Wvo.transpose(0, 2, 1)))
    d_vo_t = et.DeviceBuffer.empty((B, nh, S, N), np.float16)
    et.check(et.lib().et_linear_vo_t_f16(d_wt.ptr, up(et, bvo).ptr, d_x.ptr, d_vo_t.ptr, B, S, H, N, nh, None))
    assert Hn.max_abs(d_vo_t.numpy(), want_vo) <= 4e-3
    d_p = et.DeviceBuffer.empty((T, nh * S), np.float16)
    d_out = et.DeviceBuffer.empty((T, H), np.float16)
    et.check(et.lib().et_fill_f16(d_out.ptr, T * H, 0x7E00, None))
    et.check(et.lib().et_mha_vo_f16(d_q.ptr, d_k.ptr, H, H, d_vo.ptr, d_p.ptr, d_out.ptr, up(et, c["bo"]).ptr,
                                    None if col_id is None else up(et, col_id).ptr, None, up(et, lens).ptr, B, S, nh, hd,
                                    N, H, 1 / math.sqrt(hd), 0, None))
    Wvo_full, bvo_full = c["Wvo"].astype(np.float32), c["bvo"].astype(np.float32)
    if pruned:  # pruned columns of W_VO are zero; their outputs carry b_O alone
        m = np.zeros(H, bool); m[col_id] = True
        Wvo_full, bvo_full = Wvo_full * m, bvo_full * m
    want = L.fused_vo_attention(Hn.f32(x), Hn.f32(x), Hn.f32(x), Hn.f32(c["Wq"]), Hn.f32(c["bq"]), Hn.f32(c["Wk"]),
                                Hn.f32(c["bk"]), torch.from_numpy(Wvo_full), torch.from_numpy(bvo_full), Hn.f32(c["bo"]),
                                nh, B, lens=lens, store=torch.float16).numpy()
    # the projection key-contiguous and without bias, for the kernel that keeps the probabilities on chip
    d_vok = et.DeviceBuffer.empty((B, nh, N, S), np.float16)
    et.check(et.lib().et_linear_vo_keys_f16(d_wt.ptr, d_x.ptr, d_vok.ptr, B, S, H, N, nh, None))
    want_vok = (x.astype(np.float32).reshape(B, 1, S, H) @ Wvo.astype(np.float32)[None]).transpose(0, 1, 3, 2)
    assert Hn.max_abs(d_vok.numpy(), want_vok.astype(np.float16)) <= 4e-3
    d_otf = et.DeviceBuffer.empty((T, H), np.float16)
    et.check(et.lib().et_fill_f16(d_otf.ptr, T * H, 0x7E00, None))
    et.check(et.lib().et_mha_vo_otf_f16(d_q.ptr, d_k.ptr, H, H, d_vok.ptr, up(et, bvo).ptr, d_otf.ptr, up(et, c["bo"]).ptr,
                                        None if col_id is None else up(et, col_id).ptr, None, up(et, lens).ptr, B, S, nh,
                                        hd, N, H, 1 / math.sqrt(hd), 0, None))
    for got in (d_out.numpy(), d_otf.numpy()):
        assert Hn.max_abs(got, want) <= 6e-3
        if pruned:
            dead = np.setdiff1d(np.arange(H), col_id)
            assert np.array_equal(got[:, dead], np.broadcast_to(c["bo"][dead], (T, len(dead))))
    # both kernels round the same fp16 probabilities; they differ in the order of the fp32 sums and in
    # where the projection's bias is added
    assert Hn.max_abs(d_out.numpy(), d_otf.numpy()) <= 6e-3  # an fp16 ulp at the largest outputs


@pytest.mark.parametrize("B,S,H,nh", [(2, 192, 128, 2), (1, 64, 384, 12), (3, 80, 128, 8), (12, 256, 192, 3)])
@pytest.mark.parametrize("causal,masked", [(True, False), (False, True), (True, True)])
def test_vo_attention_on_chip_masks(et, causal, masked, B, S, H, nh):
    """Causal flag and additive mask of the on-chip VO attention against the oracle, in each of the
    kernel's forms (a wave per head for up to 4, 8 and more heads; the large-grid form)."""
    T, hd = B * S, H // nh
    q, k = Hn.randn((T, H), 40), Hn.randn((T, H), 41)
    vo = (Hn.randn((B, nh, S, H), 42).astype(np.float32) * 0.25).astype(np.float16)
    bo = Hn.randn((H,), 43)
    mask = None
    if masked:
        mask = (Hn.randn((S, S), 44).astype(np.float32) * 2).astype(np.float16)
        mask[:, 5] = -np.inf
    d_out = et.DeviceBuffer.empty((T, H), np.float16)
    vo_keys = np.ascontiguousarray(vo.transpose(0, 1, 3, 2))  # [B][nh][N][S]
    et.check(et.lib().et_mha_vo_otf_f16(up(et, q).ptr, up(et, k).ptr, H, H, up(et, vo_keys).ptr, None, d_out.ptr, up(et, bo).ptr,
                                        None, None if mask is None else up(et, mask).ptr, None, B, S, nh, hd, H, H,
                                        1 / math.sqrt(hd), et.MHA_CAUSAL if causal else 0, None))
    # the oracle's attention with V = VO_h gives softmax_h VO_h per head; the heads are summed here
    want = np.zeros((T, H), np.float32)
    for h in range(nh):
        sl = slice(h * hd, (h + 1) * hd)
        v_h = vo[:, h].reshape(T, H)
        z = L.mha(Hn.f32(q[:, sl]), Hn.f32(k[:, sl]), Hn.f32(v_h), 1, B, scale=1 / math.sqrt(hd),
                  mask=None if mask is None else Hn.f32(mask), causal=causal, store=None)
        want += z.numpy()
    want += bo.astype(np.float32)
    assert Hn.max_abs(d_out.numpy(), want) <= 6e-3


def _random_vo_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        nh, hd = int(rng.integers(1, 13)), 16 * int(rng.integers(1, 9))
        cases.append((int(rng.integers(1, 5)), 16 * int(rng.integers(1, 21)), nh, hd, 16 * int(rng.integers(1, 25)),
                      int(rng.integers(0, 4)), int(rng.integers(1, 1 << 30))))
    return cases


@pytest.mark.parametrize("B,S,nh,hd,N,kind,seed", _random_vo_cases(20, 20211118))
def test_vo_attention_on_chip_random_shapes(et, B, S, nh, hd, N, kind, seed):
    """Seeded random shapes of the on-chip VO attention (any number of heads up to 12, head sizes 16 to 128,
    output widths that leave a partial column slice): plain, padded, causal, additively masked with padding."""
    rng = np.random.default_rng(seed)
    T, H = B * S, nh * hd
    q, k = Hn.randn((T, H), seed & 0xFFF), Hn.randn((T, H), (seed & 0xFFF) + 1)
    vo = (Hn.randn((B, nh, S, N), 42).astype(np.float32) * 0.25).astype(np.float16)
    bvo, bo = Hn.randn((nh, N), 45, 0.1), Hn.randn((N,), 43)
    lens = rng.integers(0, S + 1, B).astype(np.int32) if kind in (1, 3) else None
    mask = (rng.standard_normal((S, S)) * 2).astype(np.float16) if kind == 3 else None
    d_out = et.DeviceBuffer.empty((T, N), np.float16)
    vo_keys = np.ascontiguousarray(vo.transpose(0, 1, 3, 2))  # [B][nh][N][S]
    et.check(et.lib().et_mha_vo_otf_f16(up(et, q).ptr, up(et, k).ptr, H, H, up(et, vo_keys).ptr, up(et, bvo).ptr, d_out.ptr,
                                        up(et, bo).ptr, None, None if mask is None else up(et, mask).ptr,
                                        None if lens is None else up(et, lens).ptr, B, S, nh, hd, N, N,
                                        1 / math.sqrt(hd), et.MHA_CAUSAL if kind == 2 else 0, None))
    want = np.zeros((T, N), np.float32)
    for h in range(nh):
        sl = slice(h * hd, (h + 1) * hd)
        v_h = (vo[:, h].astype(np.float32) + bvo[h].astype(np.float32)).reshape(T, N)
        z = L.mha(Hn.f32(q[:, sl]), Hn.f32(k[:, sl]), torch.from_numpy(v_h), 1, B, scale=1 / math.sqrt(hd),
                  mask=None if mask is None else Hn.f32(mask), lens=lens, causal=kind == 2, store=None)
        want += z.numpy()
    want += bo.astype(np.float32)
    got = d_out.numpy().astype(np.float32)
    if lens is not None:  # rows past a sequence's length are padding: not compared
        for b in range(B):
            got[b * S + lens[b]:(b + 1) * S] = 0
            want[b * S + lens[b]:(b + 1) * S] = 0
    assert Hn.max_abs(got, want) <= 6e-3 * max(1.0, float(np.abs(want).max()) / 4)


def test_vo_attention_on_chip_rejects_bad_shapes(et):
    d = et.DeviceBuffer.empty((64, 64), np.float16)
    call = lambda **kw: et.lib().et_mha_vo_otf_f16(d.ptr, d.ptr, kw.get("ld", 64), 64, d.ptr, None, d.ptr, None, None, None, None,
                                                   1, kw.get("S", 16), 1, kw.get("hd", 64), kw.get("N", 64),
                                                   kw.get("W", 64), 0.125, kw.get("flags", 0), None)
    assert call() == et.ET_OK
    for bad in (dict(S=24), dict(hd=40), dict(N=40, W=40), dict(N=32, W=64), dict(ld=32), dict(flags=8)):
        assert call(**bad) in (et.ET_ERR_INVALID_ARG, et.ET_ERR_UNSUPPORTED), bad


@pytest.mark.parametrize("B,S,nh,hd,keep", [(2, 128, 12, 64, 0.75), (1, 48, 4, 32, 0.5), (1, 272, 2, 64, 0.25)])
def test_compact_v_attention(et, B, S, nh, hd, keep):
    """Attention-aware pruning: V arrives compact with col_id / head_ptr; Z is full width with
    zeros in pruned columns and equals dense attention over V with the pruned columns zeroed."""
    H, T = nh * hd, B * S
    q, k = Hn.randn((T, H), 30), Hn.randn((T, H), 31)
    col_id = F.gen_row_ids(H, 1 - keep, seed=32)  # surviving V columns, ascending (row ids of W_V)
    hp = F.head_ptr(col_id, len(col_id), nh, H)
    assert hp[-1] == len(col_id)
    vc = Hn.randn((T, len(col_id)), 33)
    lens = np.array([S, S - 7][:B], np.int32)
    d_z = et.DeviceBuffer.empty((T, H), np.float16)
    et.check(et.lib().et_fill_f16(d_z.ptr, T * H, 0x7E00, None))
    et.check(et.lib().et_mha_compactv_f16(up(et, q).ptr, up(et, k).ptr, up(et, vc).ptr, H, H, len(col_id),
                                          up(et, col_id).ptr, up(et, hp).ptr, len(col_id), d_z.ptr, H, None,
                                          up(et, lens).ptr, B, S, nh, hd, hd, 1 / math.sqrt(hd), 0, None))
    v_full = np.zeros((T, H), np.float16)
    v_full[:, col_id] = vc
    want = L.mha(Hn.f32(q), Hn.f32(k), Hn.f32(v_full), nh, B, lens=lens, store=torch.float16).numpy()
    got = d_z.numpy()
    assert Hn.max_abs(got, want) <= 2e-3
    dead = np.setdiff1d(np.arange(H), col_id)
    assert np.all(got[:, dead] == 0)


def _random_compact_cases(n, seed):
    rng = np.random.default_rng(seed)
    return [(int(rng.integers(1, 5)), 16 * int(rng.integers(1, 25)), int(rng.integers(1, 13)), 16 * int(rng.integers(1, 9)),
             float(rng.choice([0.25, 0.5, 0.75, 0.9])), bool(rng.integers(0, 2)), int(rng.integers(1, 1 << 30)))
            for _ in range(n)]


@pytest.mark.parametrize("B,S,nh,hd,keep,causal,seed", _random_compact_cases(20, 20211119))
def test_compact_v_attention_random_shapes(et, B, S, nh, hd, keep, causal, seed):
    """Seeded random shapes of the compact-V attention: surviving columns of every count per head (none, a
    few, runs that do and do not start on multiples of 8), right padding, causal or not."""
    rng = np.random.default_rng(seed)
    H, T = nh * hd, B * S
    q, k = Hn.randn((T, H), seed & 0xFFF), Hn.randn((T, H), (seed & 0xFFF) + 1)
    col_id = F.gen_row_ids(H, 1 - keep, seed=seed)
    hp = F.head_ptr(col_id, len(col_id), nh, H)
    vc = Hn.randn((T, max(len(col_id), 1)), 33)[:, :len(col_id)]
    vc = np.ascontiguousarray(vc)
    lens = rng.integers(0, S + 1, B).astype(np.int32)
    d_z = et.DeviceBuffer.empty((T, H), np.float16)
    et.check(et.lib().et_fill_f16(d_z.ptr, T * H, 0x7E00, None))
    et.check(et.lib().et_mha_compactv_f16(up(et, q).ptr, up(et, k).ptr, up(et, vc).ptr, H, H, len(col_id),
                                          up(et, col_id).ptr, up(et, hp).ptr, len(col_id), d_z.ptr, H, None,
                                          up(et, lens).ptr, B, S, nh, hd, hd, 1 / math.sqrt(hd),
                                          et.MHA_CAUSAL if causal else 0, None))
    v_full = np.zeros((T, H), np.float16)
    v_full[:, col_id] = vc
    want = L.mha(Hn.f32(q), Hn.f32(k), Hn.f32(v_full), nh, B, lens=lens, causal=causal, store=torch.float16).numpy()
    got = d_z.numpy()
    for b in range(B):  # rows past a sequence's length are padding: not compared
        got[b * S + lens[b]:(b + 1) * S] = 0
        want[b * S + lens[b]:(b + 1) * S] = 0
    assert Hn.max_abs(got, want) <= 2e-3
    dead = np.setdiff1d(np.arange(H), col_id)
    assert np.all(got[:, dead] == 0)
