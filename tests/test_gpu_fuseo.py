"""Attention and the tile-sparse output projection in one launch (et_mha_fuseo_f16) against the oracle's
attention followed by its Linear (Attention/kernel_fuseO.cu:138-290 computes the same two steps), and against
the two separate launches of this library."""
import math

import numpy as np
import pytest
import torch

from oracle import layers as L
from tests import harness as Hn
from tests.harness import up

pytestmark = pytest.mark.gpu


def run_fuseo(et, B, S, nh, hd, emdim, sp, seed, lens=None, causal=False, mask=None, waves=None, bias=True,
              dead_block_rows=()):
    H = nh * hd
    T = B * S
    q, k, v = Hn.randn((T, H), seed), Hn.randn((T, H), seed + 1), Hn.randn((T, H), seed + 2)
    dq, dk, dv = up(et, q), up(et, k), up(et, v)
    w = Hn.BsrWeight(emdim, H, sp, seed=seed + 3, std=0.05, bias_std=0.1 if bias else 0.0,
                     dead_block_rows=dead_block_rows).upload(et)
    d_z = et.DeviceBuffer.empty((T, H), np.float16)
    d_out = et.DeviceBuffer.empty((T, emdim), np.float16)
    et.check(et.lib().et_fill_f16(d_z.ptr, T * H, 0x7E00, None))
    et.check(et.lib().et_fill_f16(d_out.ptr, T * emdim, 0x7E00, None))
    d_lens = up(et, np.asarray(lens, np.int32)) if lens is not None else None
    d_mask = up(et, mask.astype(np.float16)) if mask is not None else None
    flags = et.MHA_CAUSAL if causal else 0
    scale = 1.0 / math.sqrt(hd)
    et.mha_fuseo(dq, dk, dv, H, H, H, d_z, H, d_mask, d_lens, B, S, nh, hd, scale, flags, w.d_row_ptr, w.d_col_idx,
                 w.d_tiles, w.d_bias if bias else None, d_out, emdim, waves=waves)
    z_got, out_got = d_z.numpy(), d_out.numpy()
    # the two launches the one replaces
    d_z2 = et.DeviceBuffer.empty((T, H), np.float16)
    d_out2 = et.DeviceBuffer.empty((T, emdim), np.float16)
    et.mha_fused(dq, dk, dv, H, H, H, d_z2, H, d_mask, d_lens, B, S, nh, hd, scale, flags)
    w.forward(et, d_z2, d_out2, T, 0)
    z_two, out_two = d_z2.numpy(), d_out2.numpy()
    z_want = L.mha(Hn.f32(q), Hn.f32(k), Hn.f32(v), nh, B, mask=None if mask is None else Hn.f32(mask), lens=lens,
                   causal=causal, store=torch.float16)
    out_want = L.linear(z_want.float(), Hn.f32(w.dense), Hn.f32(w.bias) if bias else None, None, torch.float16)
    return (z_got, out_got), (z_two, out_two), (z_want.numpy(), out_want.numpy())


def compare(B, S, lens, got, two, want):
    z_got, out_got = (a.copy() for a in got)
    z_two, out_two = (a.copy() for a in two)
    z_want, out_want = (a.copy() for a in want)
    if lens is not None:  # rows past a sequence's length are padding: not compared
        for b in range(B):
            for a in (z_got, out_got, z_two, out_two, z_want, out_want):
                a[b * S + lens[b]:(b + 1) * S] = 0
    assert np.isfinite(z_got).all() and np.isfinite(out_got).all()
    # the attention part is the same code: bit-identical to the separate launch
    assert np.array_equal(z_got, z_two)
    assert Hn.max_abs(z_got, z_want) <= 2e-3
    # the projection: fp16 rounding of |out| < 8 plus the accumulation order; Z itself within 2e-3
    assert Hn.max_abs(out_got, out_two) <= 8e-3
    assert Hn.max_abs(out_got, out_want) <= 1.2e-2


FUSEO_CASES = [
    # B, S, nh, hd, emdim, sparsity, waves
    (1, 128, 12, 64, 768, 0.8, None),   # the reference kernel's case: one sequence of BERT-base
    (8, 128, 12, 64, 768, 0.8, None),   # the benchmark's batch
    (8, 128, 12, 64, 768, 0.8, 2),
    (8, 128, 12, 64, 768, 0.8, 1),
    (1, 384, 12, 64, 768, 0.9, None),
    (2, 64, 16, 64, 1024, 0.9, None),   # BERT-large heads
    (3, 48, 4, 32, 256, 0.5, None),     # 48 tokens: one wave per workgroup
    (2, 96, 5, 16, 208, 0.3, None),     # 80-wide Z, 13 block-rows
    (1, 128, 4, 128, 512, 0.0, None),   # every tile kept, 128-wide heads
    (2, 80, 3, 48, 144, 0.5, 4),        # strips that end past the sequence (80 = 64 + 16)
    (1, 32, 2, 72, 160, 0.4, None),     # head size between the kernel's sizes
]


@pytest.mark.parametrize("B,S,nh,hd,emdim,sp,waves", FUSEO_CASES)
def test_fuseo_matches_oracle_and_two_launches(et, B, S, nh, hd, emdim, sp, waves):
    got, two, want = run_fuseo(et, B, S, nh, hd, emdim, sp, seed=31, waves=waves)
    compare(B, S, None, got, two, want)


@pytest.mark.parametrize("kind", ["padded", "causal", "masked"])
@pytest.mark.parametrize("waves", [None, 1])
def test_fuseo_masks(et, kind, waves):
    B, S, nh, hd, emdim = 4, 128, 12, 64, 768
    rng = np.random.default_rng(5)
    lens = np.array([128, 77, 0, 16], np.int32) if kind in ("padded", "masked") else None
    mask = (rng.standard_normal((S, S)) * 2.0).astype(np.float16).astype(np.float32) if kind == "masked" else None
    got, two, want = run_fuseo(et, B, S, nh, hd, emdim, 0.8, seed=77, lens=lens, causal=kind == "causal", mask=mask,
                               waves=waves)
    compare(B, S, lens, got, two, want)


def test_fuseo_empty_block_rows_no_bias_and_repeat(et):
    """Block-rows without tiles give zeros (no bias); the arrival counts are back at zero after every launch, so
    a second and third call on other shapes see a clean state."""
    for B, S in ((2, 64), (1, 128), (5, 16)):
        got, two, want = run_fuseo(et, B, S, 4, 64, 256, 0.7, seed=3 + B, bias=False, dead_block_rows=(0, 7, 15))
        compare(B, S, None, got, two, want)
        assert not got[1][:, :16].any() and not got[1][:, 112:128].any()


def test_fuseo_rejects_what_it_cannot_do(et):
    lib = et.lib()
    d = et.DeviceBuffer.empty((16, 256), np.float16)
    rp = up(et, np.zeros(17, np.int32))
    args = lambda **kw: dict(dict(B=1, S=16, nh=4, hd=64, emdim=256), **kw)

    def call(B, S, nh, hd, emdim):
        return lib.et_mha_fuseo_f16(d.ptr, d.ptr, d.ptr, nh * hd, nh * hd, nh * hd, d.ptr, nh * hd, None, None, B, S,
                                    nh, hd, 0.125, 0, rp.ptr, rp.ptr, d.ptr, None, d.ptr, emdim, None)
    assert call(**args(S=24)) == et.ET_ERR_UNSUPPORTED          # S not a multiple of 16
    assert call(**args(hd=200, nh=1)) == et.ET_ERR_UNSUPPORTED  # head wider than 128
    assert call(**args(emdim=200)) == et.ET_ERR_UNSUPPORTED
    assert call(**args(B=20000)) == et.ET_ERR_UNSUPPORTED       # more strips than arrival counts
    assert call(**args(B=0)) == et.ET_OK


def test_fuseo_interleaved_qkv_and_strided_z(et):
    """Q, K and V as column slices of one [T x 3H] buffer and Z inside a wider buffer (row stride H + 64): the
    projection reads Z through its stride; the columns beside Z stay untouched."""
    B, S, nh, hd, emdim = 3, 64, 6, 32, 192
    H, T = nh * hd, B * S
    qkv = Hn.randn((T, 3 * H), 41)
    d_qkv = up(et, qkv)
    w = Hn.BsrWeight(emdim, H, 0.6, seed=45, std=0.05, bias_std=0.1).upload(et)
    ldz = H + 64
    zbuf = np.full((T, ldz), 7.0, np.float16)
    d_z = up(et, zbuf)
    d_out = et.DeviceBuffer.empty((T, emdim), np.float16)
    et.mha_fuseo(d_qkv.ptr, d_qkv.offset(2 * H), d_qkv.offset(4 * H), 3 * H, 3 * H, 3 * H, d_z, ldz, None, None, B, S, nh,
                 hd, 1.0 / math.sqrt(hd), 0, w.d_row_ptr, w.d_col_idx, w.d_tiles, w.d_bias, d_out, emdim)
    q, k, v = qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:]
    z_want = L.mha(Hn.f32(q), Hn.f32(k), Hn.f32(v), nh, B, store=torch.float16)
    out_want = L.linear(z_want.float(), Hn.f32(w.dense), Hn.f32(w.bias), None, torch.float16)
    z_got = d_z.numpy()
    assert Hn.max_abs(z_got[:, :H], z_want.numpy()) <= 2e-3
    assert (z_got[:, H:] == 7.0).all()
    assert Hn.max_abs(d_out.numpy(), out_want.numpy()) <= 1.2e-2


def _random_fuseo_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        S = 16 * int(rng.integers(1, 17))
        B, nh = int(rng.integers(1, 6)), int(rng.integers(1, 9))
        hd = 8 * int(rng.integers(1, 17))
        while (nh * hd) % 16:
            hd += 8
        emdim = 16 * int(rng.integers(1, 40))
        kind = int(rng.integers(0, 3))  # 0 plain, 1 right padding, 2 causal
        cases.append((B, S, nh, hd, emdim, round(float(rng.uniform(0.0, 0.95)), 2), kind, int(rng.integers(1, 1 << 20))))
    return cases


@pytest.mark.parametrize("B,S,nh,hd,emdim,sp,kind,seed", _random_fuseo_cases(16, 20211117))
def test_fuseo_random_shapes(et, B, S, nh, hd, emdim, sp, kind, seed):
    rng = np.random.default_rng(seed)
    lens = rng.integers(0, S + 1, B).astype(np.int32) if kind == 1 else None
    got, two, want = run_fuseo(et, B, S, nh, hd, emdim, sp, seed=seed & 0xFFFF, lens=lens, causal=kind == 2,
                               waves=[None, 1, 2, 4][seed % 4] if (S // 16) % 4 == 0 else None)
    compare(B, S, lens, got, two, want)
