"""The QKV projection inside the attention kernel (et_qkv_heads_pack_create, et_norm_qkv_mha_f32in): one launch
that normalises the previous layer's binary32 sum with its row statistics, projects Q, K and V of a head through
the tile-sparse W_qkv and runs the fused attention on them — against the oracle (LayerNorm -> Linear -> attention)
and against the two launches it replaces."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

from tests import harness as Hn
from tests.harness import L, up

pytestmark = pytest.mark.gpu

H, NH, HD = 768, 12, 64

CASES = [
    # B, S, sparsity, groups of row statistics, kind (0 plain, 1 right padding, 2 causal, 3 additive mask + padding)
    (8, 128, 0.8, 4, 0),
    (8, 128, 0.8, 16, 1),
    (3, 64, 0.8, 4, 1),
    (2, 48, 0.5, 1, 2),
    (9, 128, 0.9, 8, 3),
    (1, 16, 0.95, 2, 0),
    # the attention-block configuration of the benchmark: batch 1 / 4 / 16, 128 tokens, right padding in [64, 128]
    (1, 128, 0.8, 8, 1),
    (4, 128, 0.8, 8, 1),
    (16, 128, 0.8, 8, 1),
]


@pytest.mark.parametrize("folded", [False, True])
@pytest.mark.parametrize("B,S,sp,groups,kind", CASES)
def test_norm_qkv_mha(et, B, S, sp, groups, kind, folded):
    """folded: the pack holds W diag(gamma) and bias + W beta (et_qkv_heads_pack_create_folded) and the launch is given
    neither gamma, beta nor the bias."""
    lib = et.lib()
    T = B * S
    w = Hn.BsrWeight(3 * H, H, sp, seed=171, bias_std=0.05).upload(et)
    v32 = Hn.randn((T, H), 172, 1.5, np.float32) + 0.3
    gamma = (1 + Hn.randn((H,), 173, 0.1, np.float32)).astype(np.float16)
    beta = Hn.randn((H,), 174, 0.1)
    # row statistics as a producer leaves them: (sum, sum of squares) per contiguous group of columns
    bounds = np.linspace(0, H, groups + 1).astype(int)
    stats = np.zeros((groups, T, 2), np.float32)
    for gi in range(groups):
        blk = v32[:, bounds[gi]:bounds[gi + 1]].astype(np.float64)
        stats[gi, :, 0] = blk.sum(1)
        stats[gi, :, 1] = (blk * blk).sum(1)
    rng = np.random.default_rng(175)
    lens = rng.integers(S // 2, S + 1, B).astype(np.int32) if kind in (1, 3) else None
    mask = None
    if kind == 3:
        mask = np.where(rng.random((S, S)) < 0.1, -np.inf, rng.standard_normal((S, S)) * 0.5).astype(np.float16)
        mask[np.arange(S), np.arange(S)] = 0  # no row fully masked
    d_v, d_st, d_g, d_b = up(et, v32), up(et, stats), up(et, gamma), up(et, beta)
    d_lens = up(et, lens) if lens is not None else None
    d_mask = up(et, mask) if mask is not None else None
    d_fin = et.DeviceBuffer.empty((T, 2), np.float32)
    d_z = et.DeviceBuffer.empty((T, H), np.float16)
    et.check(lib.et_fill_f16(d_z.ptr, T * H, 0x7E00, None))
    assert lib.et_norm_qkv_mha_f32in_supported(B, S, H, NH, HD) == 1
    pack = C.c_void_p()
    if folded:
        et.check(lib.et_qkv_heads_pack_create_folded(w.d_row_ptr.ptr, w.d_col_idx.ptr, w.d_tiles.ptr, w.d_bias.ptr, d_g.ptr,
                                                     d_b.ptr, H, NH, C.byref(pack)))
    else:
        et.check(lib.et_qkv_heads_pack_create(w.d_row_ptr.ptr, w.d_col_idx.ptr, w.d_tiles.ptr, H, NH, C.byref(pack)))
    scale = 1.0 / math.sqrt(HD)
    flags = et.MHA_CAUSAL if kind == 2 else 0
    for _ in range(2):
        et.check(lib.et_norm_qkv_mha_f32in(pack, d_v.ptr, d_st.ptr, groups, None if folded else d_g.ptr,
                                           None if folded else d_b.ptr, 1e-5, d_fin.ptr, None if folded else w.d_bias.ptr,
                                           d_z.ptr, H, d_mask.ptr if d_mask else None, d_lens.ptr if d_lens else None, B, S,
                                           scale, flags, None))
    et.sync()
    got = d_z.numpy()
    # oracle: LayerNorm (fp32) -> fp16 operand -> Linear (fp16 result) -> attention
    y = L.layernorm(Hn.f32(v32), Hn.f32(gamma), Hn.f32(beta), 1e-5, torch.float16)
    qkv = L.linear(y, Hn.f32(w.dense), Hn.f32(w.bias), None, torch.float16)
    want = L.mha(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], NH, B, lens=lens, causal=kind == 2,
                 mask=None if mask is None else torch.from_numpy(mask.astype(np.float32)), store=torch.float16).numpy()
    live = np.ones((T, 1), bool)
    err = Hn.max_abs(got, want)
    # the two launches it replaces, on the same operands
    d_qkv = et.DeviceBuffer.empty((T, 3 * H), np.float16)
    d_z2 = et.DeviceBuffer.empty((T, H), np.float16)
    et.check(lib.et_norm_linear_bsr16_f32in(d_v.ptr, d_st.ptr, groups, d_g.ptr, d_b.ptr, 1e-5, None, None, None, w.d_row_ptr.ptr,
                                            w.d_col_idx.ptr, w.d_tiles.ptr, w.d_bias.ptr, d_qkv.ptr, T, H, 3 * H, 0, None))
    et.mha_fused(d_qkv.ptr, d_qkv.offset(2 * H), d_qkv.offset(4 * H), 3 * H, 3 * H, 3 * H, d_z2, H, d_mask, d_lens, B, S, NH, HD,
                 scale, flags, None)
    et.sync()
    err2 = Hn.max_abs(got, d_z2.numpy())
    print(f"qkv inside attention{' (folded)' if folded else ''} B={B} S={S} sp={sp}: vs oracle {err:.2e}, vs the two launches {err2:.2e}")
    assert not np.isnan(got.astype(np.float32)).any()
    assert err <= 3e-3 and err2 <= 3e-3
    fin = d_fin.numpy()
    mean = v32.astype(np.float64).mean(1)
    rstd = 1.0 / np.sqrt(v32.astype(np.float64).var(1) + 1e-5)
    assert np.max(np.abs(fin[:, 0] - mean)) <= 1e-5 and np.max(np.abs(fin[:, 1] / rstd - 1)) <= 1e-4
    et.check(lib.et_bsr16_pack_destroy(pack))


def test_norm_qkv_mha_rejects(et):
    lib = et.lib()
    assert lib.et_norm_qkv_mha_f32in_supported(8, 256, 768, 12, 64) == 0   # more than one key block
    assert lib.et_norm_qkv_mha_f32in_supported(8, 128, 1024, 16, 64) == 0  # input wider than 768
    assert lib.et_norm_qkv_mha_f32in_supported(8, 128, 768, 6, 128) == 0   # heads of 128
    w = Hn.BsrWeight(3 * 1024, 1024, 0.9, seed=176).upload(et)
    pack = C.c_void_p()
    assert lib.et_qkv_heads_pack_create(w.d_row_ptr.ptr, w.d_col_idx.ptr, w.d_tiles.ptr, 1024, 16, C.byref(pack)) == et.ET_ERR_UNSUPPORTED
