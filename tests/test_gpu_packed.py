"""The packed form of the tile-sparse Linear (et_bsr16_pack_create and the three calls that take a
pack) against the oracle: plain results in binary16 and binary32, the producer half of the split
SkipLayerNorm (binary32 sum with row sums, residual read or formed) and the consumer half (binary32
strip normalised while staged), at the automatic geometry and at forced ones."""
import ctypes as C

import numpy as np
import pytest
import torch

from tests import harness as Hn
from tests.harness import L, up

pytestmark = pytest.mark.gpu

ET_PACK_NORM_CONSUMER, ET_PACK_STATS_PRODUCER = 1, 2
ACT_NAME = {0: None, 1: "relu", 2: "gelu"}


class Pack:
    def __init__(self, et, w, T, flags=0, geom=None):
        self.et, self.lib = et, et.lib()
        self.h = C.c_void_p()
        args = (w.d_row_ptr.ptr, w.d_col_idx.ptr, w.d_tiles.ptr, T, w.inp, w.out, flags)
        if geom:
            et.check(self.lib.et_bsr16_pack_create_geom(*args, *geom, C.byref(self.h)))
        else:
            et.check(self.lib.et_bsr16_pack_create(*args, 0, C.byref(self.h)))

    def info(self):
        v = [C.c_int() for _ in range(5)]
        self.et.check(self.lib.et_bsr16_pack_info(self.h, *[C.byref(x) for x in v]))
        return dict(zip(("mt", "ngroups", "nwave", "cap", "lds"), (x.value for x in v)))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.et.check(self.lib.et_device_sync())
        self.et.check(self.lib.et_bsr16_pack_destroy(self.h))


PLAIN_CASES = [
    # T, in, out, sparsity, act, (mt, ngroups, nwave, cap) or None
    (1024, 768, 2304, 0.8, 0, None),
    (1024, 768, 768, 0.8, 0, None),
    (1024, 768, 3072, 0.8, 2, None),
    (1024, 3072, 768, 0.8, 0, None),
    (2048, 768, 768, 0.8, 1, None),
    (2048, 768, 3072, 0.9, 2, None),
    (2048, 3072, 768, 0.9, 0, None),
    (2048, 1024, 4096, 0.9, 2, None),
    (2048, 4096, 1024, 0.9, 0, None),
    (128, 768, 2304, 0.9, 0, None),
    (128, 3072, 768, 0.8, 0, None),
    (16, 128, 16, 0.0, 0, None),
    (48, 256, 32, 0.3, 2, None),          # ragged last strip of 32-row strips
    (1040, 768, 768, 0.8, 1, None),
    (256, 1024, 1024, 0.95, 0, None),     # block-rows without tiles
    (512, 768, 768, 0.8, 0, (1, 4, 7, 12)),
    (512, 768, 768, 0.8, 2, (2, 3, 16, 8)),
    (1024, 768, 3072, 0.8, 0, (2, 8, 7, 24)),
    (64, 384, 208, 0.5, 1, (2, 13, 1, 12)),  # one block-row per group, one wave
    (64, 384, 208, 0.5, 1, (1, 1, 4, 24)),
]


@pytest.mark.parametrize("T,inp,out,sp,act,geom", PLAIN_CASES)
def test_linear_bsr16_packed(et, T, inp, out, sp, act, geom):
    lib = et.lib()
    w = Hn.BsrWeight(out, inp, sp, seed=131, bias_std=0.1).upload(et)
    x = Hn.randn((T, inp), 132)
    d_x = up(et, x)
    with Pack(et, w, T, 0, geom) as pk:
        g = pk.info()
        d_y16 = et.DeviceBuffer.empty((T, out), np.float16)
        d_y32 = et.DeviceBuffer.empty((T, out), np.float32)
        et.check(lib.et_fill_f16(d_y16.ptr, T * out, 0x7E00, None))
        et.check(lib.et_linear_bsr16_packed_f16(pk.h, w.d_bias.ptr, d_x.ptr, d_y16.ptr, None, T, act, None))
        et.check(lib.et_linear_bsr16_packed_f16(pk.h, w.d_bias.ptr, d_x.ptr, None, d_y32.ptr, T, act, None))
        want32 = L.linear(Hn.f32(x), Hn.f32(w.dense), Hn.f32(w.bias), ACT_NAME[act], None).numpy()
        want16 = L.linear(Hn.f32(x), Hn.f32(w.dense), Hn.f32(w.bias), ACT_NAME[act], torch.float16).numpy()
        e16, e32 = Hn.max_abs(d_y16.numpy(), want16), Hn.max_abs(d_y32.numpy(), want32)
        print(f"packed T={T} in={inp} out={out} sp={sp} {g}: max-abs fp16 {e16:.2e} fp32 {e32:.2e}")
        assert e16 <= 4e-3
        assert e32 <= 5e-5 * max(1.0, float(np.abs(want32).max()))
        # without a bias, and with fewer rows than the pack was built for
        T2 = 16 * max(1, T // 48)
        d_y = et.DeviceBuffer.empty((T2, out), np.float16)
        et.check(lib.et_linear_bsr16_packed_f16(pk.h, None, d_x.ptr, d_y.ptr, None, T2, 0, None))
        want = L.linear(Hn.f32(x[:T2]), Hn.f32(w.dense), None, None, torch.float16).numpy()
        assert Hn.max_abs(d_y.numpy(), want) <= 4e-3


ET_PACK_ROW_LOOP = 4
ROW_LOOP_CASES = [
    # T, in, out, sparsity, act
    (2048, 768, 3072, 0.8, 2),     # 32-row strips, several strips per workgroup
    (4112, 768, 768, 0.8, 0),      # a last strip of 16 rows
    (16384, 768, 2304, 0.8, 0),    # the large-batch QKV projection
    (96, 128, 64, 0.5, 1),         # fewer strips than compute units, one group
    (1024, 1024, 768, 0.9, 1),
    (528, 1536, 256, 0.8, 2),      # 16-row strips (three 32-row strips of 1536 values do not fit the LDS)
    (160, 768, 768, 0.97, 0),      # block-rows without tiles
    (64, 256, 4096, 0.0, 0),       # dense pattern, many groups
]


@pytest.mark.parametrize("T,inp,out,sp,act", ROW_LOOP_CASES)
def test_linear_bsr16_row_loop(et, T, inp, out, sp, act):
    """The pack for many token rows (ET_PACK_ROW_LOOP): weights resident in registers, strips double-buffered,
    results straight from the accumulators — the values of et_linear_bsr16_f16."""
    lib = et.lib()
    w = Hn.BsrWeight(out, inp, sp, seed=151, bias_std=0.1).upload(et)
    x = Hn.randn((T, inp), 152)
    d_x = up(et, x)
    with Pack(et, w, T, ET_PACK_ROW_LOOP) as pk:
        g = pk.info()
        d_y = et.DeviceBuffer.empty((T, out), np.float16)
        for rep in range(2):  # the second launch finds the first one's results in place: every element is written again
            et.check(lib.et_fill_f16(d_y.ptr, T * out, 0x7E00, None))
            et.check(lib.et_linear_bsr16_packed_f16(pk.h, w.d_bias.ptr, d_x.ptr, d_y.ptr, None, T, act, None))
        want = L.linear(Hn.f32(x), Hn.f32(w.dense), Hn.f32(w.bias), ACT_NAME[act], torch.float16).numpy()
        got = d_y.numpy()
        err = Hn.max_abs(got, want)
        print(f"row loop T={T} in={inp} out={out} sp={sp} {g}: max-abs {err:.2e}")
        assert not np.isnan(got.astype(np.float32)).any()
        assert err <= 4e-3
        # no bias, fewer rows than the pack was built for (a multiple of 16 that ends inside a 32-row strip)
        T2 = 16 * max(1, T // 48)
        d_y2 = et.DeviceBuffer.empty((T2, out), np.float16)
        et.check(lib.et_linear_bsr16_packed_f16(pk.h, None, d_x.ptr, d_y2.ptr, None, T2, 0, None))
        want = L.linear(Hn.f32(x[:T2]), Hn.f32(w.dense), None, None, torch.float16).numpy()
        assert Hn.max_abs(d_y2.numpy(), want) <= 4e-3
        # binary32 results: the accumulator plus bias, activated, unrounded (twice in a row, then a ragged row count)
        d_y32 = et.DeviceBuffer.empty((T, out), np.float32)
        want32 = L.linear(Hn.f32(x), Hn.f32(w.dense), Hn.f32(w.bias), ACT_NAME[act], None).numpy()
        for rep in range(2):
            et.check(lib.et_memset(d_y32.ptr, 0xFF, T * out * 4, None))  # NaN patterns: every element must be written
            et.check(lib.et_linear_bsr16_packed_f16(pk.h, w.d_bias.ptr, d_x.ptr, None, d_y32.ptr, T, act, None))
        got32 = d_y32.numpy()
        assert not np.isnan(got32).any()
        assert Hn.max_abs(got32, want32) <= 2e-3
        d_y32b = et.DeviceBuffer.empty((T2, out), np.float32)
        et.check(lib.et_memset(d_y32b.ptr, 0xFF, T2 * out * 4, None))
        et.check(lib.et_linear_bsr16_packed_f16(pk.h, w.d_bias.ptr, d_x.ptr, None, d_y32b.ptr, T2, act, None))
        assert np.array_equal(d_y32b.numpy(), got32[:T2])


def test_row_loop_pack_rejects(et):
    lib = et.lib()
    w = Hn.BsrWeight(64, 1664, 0.5, seed=153).upload(et)  # in above 1536
    h = C.c_void_p()
    args = (w.d_row_ptr.ptr, w.d_col_idx.ptr, w.d_tiles.ptr, 64, w.inp, w.out)
    assert lib.et_bsr16_pack_create(*args, ET_PACK_ROW_LOOP, 0, C.byref(h)) == et.ET_ERR_UNSUPPORTED
    w2 = Hn.BsrWeight(64, 256, 0.5, seed=154).upload(et)
    args = (w2.d_row_ptr.ptr, w2.d_col_idx.ptr, w2.d_tiles.ptr, 64, w2.inp, w2.out)
    assert lib.et_bsr16_pack_create(*args, ET_PACK_ROW_LOOP | ET_PACK_STATS_PRODUCER, 0, C.byref(h)) == et.ET_ERR_INVALID_ARG
    assert lib.et_bsr16_pack_create(*args, ET_PACK_ROW_LOOP, 12, C.byref(h)) == et.ET_ERR_INVALID_ARG  # own geometry


def test_linear_bsr16_packed_closed_form_and_tile_order(et):
    """All-ones weights and inputs give 16 * tiles-in-row + bias exactly (the closed form of the
    reference's driver, Linear/test/test_tile.cu), whatever the order of the tiles in a row."""
    lib = et.lib()
    T, inp, out = 64, 512, 256
    w = Hn.BsrWeight(out, inp, 0.7, seed=133)
    w.tiles = np.ones_like(w.tiles)
    w.bias = np.full(out, 0.5, np.float16)
    w.upload(et)
    d_x = up(et, np.ones((T, inp), np.float16))
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    with Pack(et, w, T) as pk:
        et.check(lib.et_linear_bsr16_packed_f16(pk.h, w.d_bias.ptr, d_x.ptr, d_y.ptr, None, T, 0, None))
    per_row = np.diff(w.row_ptr).astype(np.float32)
    want = np.repeat(16.0 * per_row + 0.5, 16)[None, :].repeat(T, 0)
    assert np.array_equal(d_y.numpy().astype(np.float32), want)


SPLIT_CASES = [
    # T, n_in (producer input), n_mid (normalised width), n_out, sparsity, act
    (1024, 768, 768, 3072, 0.8, 2),     # O projection -> FFN up
    (1024, 3072, 768, 2304, 0.8, 0),    # FFN down -> QKV
    (2048, 4096, 1024, 4096, 0.9, 2),   # BERT-large shapes
    (2048, 1024, 1024, 3072, 0.9, 0),
    (128, 768, 768, 3072, 0.9, 2),
    (128, 3072, 768, 2304, 0.9, 0),
    (48, 256, 512, 128, 0.5, 1),
    (272, 384, 768, 896, 0.5, 0),
]


@pytest.mark.parametrize("T,n_in,n_mid,n_out,sp,act", SPLIT_CASES)
def test_split_layernorm_packed(et, T, n_in, n_mid, n_out, sp, act):
    """Producer (binary32 sum + row sums) and consumer (strip normalised while staged) through packs:
    the values of et_linear_bsr16_resid_stats_f32 and et_norm_linear_bsr16_f32in."""
    lib = et.lib()
    w1 = Hn.BsrWeight(n_mid, n_in, sp, seed=141, bias_std=0.05).upload(et)
    w2 = Hn.BsrWeight(n_out, n_mid, sp, seed=144, bias_std=0.05).upload(et)
    x = Hn.randn((T, n_in), 147)
    resid = Hn.randn((T, n_mid), 148, 1.0, np.float32)
    gamma = (1 + Hn.randn((n_mid,), 149, 0.1, np.float32)).astype(np.float16)
    beta = Hn.randn((n_mid,), 150, 0.1)
    d_x, d_resid, d_g, d_b = up(et, x), up(et, resid), up(et, gamma), up(et, beta)
    d_v = et.DeviceBuffer.empty((T, n_mid), np.float32)
    d_stats = et.DeviceBuffer.empty((16, T, 2), np.float32)
    groups = C.c_int(0)
    with Pack(et, w1, T, ET_PACK_STATS_PRODUCER) as p1, Pack(et, w2, T, ET_PACK_NORM_CONSUMER) as p2:
        print(f"producer {p1.info()} consumer {p2.info()}")
        et.check(lib.et_linear_bsr16_packed_resid_stats_f32(p1.h, w1.d_bias.ptr, d_x.ptr, d_resid.ptr, None, None, None,
                                                            None, d_v.ptr, d_stats.ptr, C.byref(groups), T, None))
        G = groups.value
        assert 1 <= G <= 16
        v = d_v.numpy()
        want_v = L.linear(Hn.f32(x), Hn.f32(w1.dense), Hn.f32(w1.bias)).numpy() + resid
        assert Hn.max_abs(v, want_v) <= 1e-4 * max(1.0, float(np.abs(want_v).max()))
        st = d_stats.numpy()[:G].astype(np.float64).sum(0)
        v64 = v.astype(np.float64)
        assert np.allclose(st[:, 0], v64.sum(1), rtol=1e-5, atol=1e-3)
        assert np.allclose(st[:, 1], (v64 * v64).sum(1), rtol=1e-5, atol=1e-3)

        d_y = et.DeviceBuffer.empty((T, n_out), np.float16)
        d_fin = et.DeviceBuffer.empty((T, 2), np.float32)
        et.check(lib.et_fill_f16(d_y.ptr, T * n_out, 0x7E00, None))
        et.check(lib.et_norm_linear_bsr16_packed_f32in(p2.h, d_v.ptr, d_stats.ptr, G, d_g.ptr, d_b.ptr, 1e-5, d_fin.ptr,
                                                       w2.d_bias.ptr, d_y.ptr, T, act, None))
        fin = d_fin.numpy().astype(np.float64)
        assert np.allclose(fin[:, 0], v64.mean(1), rtol=1e-5, atol=1e-5)
        assert np.allclose(fin[:, 1], 1 / np.sqrt(v64.var(1) + 1e-5), rtol=1e-4)
        want_ln = L.layernorm(torch.from_numpy(v), Hn.f32(gamma), Hn.f32(beta), 1e-5).numpy()
        ln16 = want_ln.astype(np.float16)
        want_y = L.linear(Hn.f32(ln16), Hn.f32(w2.dense), Hn.f32(w2.bias), ACT_NAME[act], torch.float16).numpy()
        assert Hn.max_abs(d_y.numpy(), want_y) <= 6e-3
        # without fin_out the result is the same
        d_y2 = et.DeviceBuffer.empty((T, n_out), np.float16)
        et.check(lib.et_norm_linear_bsr16_packed_f32in(p2.h, d_v.ptr, d_stats.ptr, G, d_g.ptr, d_b.ptr, 1e-5, None,
                                                       w2.d_bias.ptr, d_y2.ptr, T, act, None))
        assert np.array_equal(d_y2.numpy().view(np.uint16), d_y.numpy().view(np.uint16))

    # a second producer whose residual is the normalisation of V, formed in its epilogue from V, the
    # (mean, rstd) the consumer left and the affine vectors; and one with a binary16 residual
    w3 = Hn.BsrWeight(n_mid, n_out, sp, seed=145, bias_std=0.05).upload(et)
    d_v2 = et.DeviceBuffer.empty((T, n_mid), np.float32)
    d_v3 = et.DeviceBuffer.empty((T, n_mid), np.float32)
    d_st2 = et.DeviceBuffer.empty((16, T, 2), np.float32)
    r16 = Hn.randn((T, n_mid), 146)
    d_r16 = up(et, r16)
    with Pack(et, w3, T, ET_PACK_STATS_PRODUCER) as p3:
        et.check(lib.et_linear_bsr16_packed_resid_stats_f32(p3.h, w3.d_bias.ptr, d_y.ptr, d_v.ptr, None, d_fin.ptr, d_g.ptr,
                                                            d_b.ptr, d_v2.ptr, d_st2.ptr, C.byref(groups), T, None))
        et.check(lib.et_linear_bsr16_packed_resid_stats_f32(p3.h, w3.d_bias.ptr, d_y.ptr, None, d_r16.ptr, None, None,
                                                            None, d_v3.ptr, d_st2.ptr, C.byref(groups), T, None))
        proj = L.linear(Hn.f32(d_y.numpy()), Hn.f32(w3.dense), Hn.f32(w3.bias)).numpy()
        want_v2 = proj + want_ln
        assert Hn.max_abs(d_v2.numpy(), want_v2) <= 3e-4 * max(1.0, float(np.abs(want_v2).max()))
        want_v3 = proj + r16.astype(np.float32)
        assert Hn.max_abs(d_v3.numpy(), want_v3) <= 1e-4 * max(1.0, float(np.abs(want_v3).max()))
        st = d_st2.numpy()[: groups.value].astype(np.float64).sum(0)
        v3 = d_v3.numpy().astype(np.float64)
        assert np.allclose(st[:, 0], v3.sum(1), rtol=1e-5, atol=1e-3)


def test_pack_rejects_what_it_cannot_do(et):
    lib = et.lib()
    w = Hn.BsrWeight(64, 192, 0.5, seed=151).upload(et)
    h = C.c_void_p()
    args = (w.d_row_ptr.ptr, w.d_col_idx.ptr, w.d_tiles.ptr)
    assert lib.et_bsr16_pack_create(*args, 64, 192, 64, 0, 0, C.byref(h)) == et.ET_ERR_UNSUPPORTED  # in % 128
    assert lib.et_bsr16_pack_create(*args, 60, 192, 64, 0, 0, C.byref(h)) == et.ET_ERR_UNSUPPORTED  # T % 16
    assert lib.et_bsr16_pack_create(*args, 64, 192, 64, 8, 0, C.byref(h)) == et.ET_ERR_INVALID_ARG  # flags
    w2 = Hn.BsrWeight(64, 256, 0.5, seed=152).upload(et)
    args2 = (w2.d_row_ptr.ptr, w2.d_col_idx.ptr, w2.d_tiles.ptr)
    assert lib.et_bsr16_pack_create(*args2, 64, 256, 64, ET_PACK_NORM_CONSUMER, 0, C.byref(h)) == et.ET_ERR_UNSUPPORTED  # in < 512
    assert lib.et_bsr16_pack_create_geom(*args2, 64, 256, 64, 0, 1, 1, 1, 4, C.byref(h)) == et.ET_ERR_UNSUPPORTED  # 4 slots, 1 wave
    assert h.value is None
    # a plain pack cannot serve as a normalising consumer
    et.check(lib.et_bsr16_pack_create(*args2, 64, 256, 64, 0, 0, C.byref(h)))
    d = et.DeviceBuffer.empty((64, 256), np.float32)
    assert lib.et_norm_linear_bsr16_packed_f32in(h, d.ptr, d.ptr, 1, d.ptr, d.ptr, 1e-5, None, None, d.ptr, 64, 0,
                                                 None) == et.ET_ERR_INVALID_ARG
    et.check(lib.et_bsr16_pack_destroy(h))


def test_encoder_chain_equals_its_four_calls(et):
    """et_encoder_chain_f32 against the four packed calls it stands for (same packs, same operands):
    every buffer bit for bit, the status words clean."""
    lib = et.lib()
    T, H, FF = 1024, 768, 3072
    wo = Hn.BsrWeight(H, H, 0.8, seed=161, bias_std=0.05).upload(et)
    w1 = Hn.BsrWeight(FF, H, 0.8, seed=164, bias_std=0.05).upload(et)
    w2 = Hn.BsrWeight(H, FF, 0.8, seed=167, bias_std=0.05).upload(et)
    wq = Hn.BsrWeight(3 * H, H, 0.8, seed=170, bias_std=0.05).upload(et)
    z = up(et, Hn.randn((T, H), 173))
    resid = up(et, Hn.randn((T, H), 174, 1.0, np.float32))
    g1 = up(et, (1 + Hn.randn((H,), 175, 0.1, np.float32)).astype(np.float16))
    b1 = up(et, Hn.randn((H,), 176, 0.1))
    g2 = up(et, (1 + Hn.randn((H,), 177, 0.1, np.float32)).astype(np.float16))
    b2 = up(et, Hn.randn((H,), 178, 0.1))

    def buffers():
        return dict(V1=et.DeviceBuffer.empty((T, H), np.float32), st1=et.DeviceBuffer.empty((16, T, 2), np.float32),
                    fin1=et.DeviceBuffer.empty((T, 2), np.float32), Hh=et.DeviceBuffer.empty((T, FF), np.float16),
                    V2=et.DeviceBuffer.empty((T, H), np.float32), st2=et.DeviceBuffer.empty((16, T, 2), np.float32),
                    fin2=et.DeviceBuffer.empty((T, 2), np.float32), QKV=et.DeviceBuffer.empty((T, 3 * H), np.float16))

    def pack(w, flags):
        h = C.c_void_p()
        et.check(lib.et_bsr16_pack_create(w.d_row_ptr.ptr, w.d_col_idx.ptr, w.d_tiles.ptr, T, w.inp, w.out, flags, 12,
                                          C.byref(h)))
        return h

    po, pu, pd, pq = (pack(wo, ET_PACK_STATS_PRODUCER), pack(w1, ET_PACK_NORM_CONSUMER), pack(w2, ET_PACK_STATS_PRODUCER),
                      pack(wq, ET_PACK_NORM_CONSUMER))
    try:
        # the four calls
        a = buffers()
        g = C.c_int()
        et.check(lib.et_linear_bsr16_packed_resid_stats_f32(po, wo.d_bias.ptr, z.ptr, resid.ptr, None, None, None, None,
                                                            a["V1"].ptr, a["st1"].ptr, C.byref(g), T, None))
        g1n = g.value
        et.check(lib.et_norm_linear_bsr16_packed_f32in(pu, a["V1"].ptr, a["st1"].ptr, g1n, g1.ptr, b1.ptr, 1e-5,
                                                       a["fin1"].ptr, w1.d_bias.ptr, a["Hh"].ptr, T, 2, None))
        et.check(lib.et_linear_bsr16_packed_resid_stats_f32(pd, w2.d_bias.ptr, a["Hh"].ptr, a["V1"].ptr, None, a["fin1"].ptr,
                                                            g1.ptr, b1.ptr, a["V2"].ptr, a["st2"].ptr, C.byref(g), T, None))
        g2n = g.value
        et.check(lib.et_norm_linear_bsr16_packed_f32in(pq, a["V2"].ptr, a["st2"].ptr, g2n, g2.ptr, b2.ptr, 1e-5,
                                                       a["fin2"].ptr, wq.d_bias.ptr, a["QKV"].ptr, T, 0, None))
        # the chain
        b = buffers()
        sync = et.DeviceBuffer.from_numpy(np.zeros(288, np.uint32))
        d = et.ChainDesc()
        d.o, d.bias_o, d.Z, d.resid, d.V1, d.stats1 = po.value, wo.d_bias.ptr, z.ptr, resid.ptr, b["V1"].ptr, b["st1"].ptr
        d.up, d.bias_up, d.gamma1, d.beta1, d.eps1, d.fin1, d.H, d.act = (pu.value, w1.d_bias.ptr, g1.ptr, b1.ptr, 1e-5,
                                                                          b["fin1"].ptr, b["Hh"].ptr, 2)
        d.down, d.bias_down, d.V2, d.stats2 = pd.value, w2.d_bias.ptr, b["V2"].ptr, b["st2"].ptr
        d.qkv, d.bias_qkv, d.gamma2, d.beta2, d.eps2, d.fin2, d.QKV = (pq.value, wq.d_bias.ptr, g2.ptr, b2.ptr, 1e-5,
                                                                       b["fin2"].ptr, b["QKV"].ptr)
        d.T, d.sync = T, sync.ptr
        assert lib.et_encoder_chain_supported(C.byref(d)) == 1
        et.check(lib.et_encoder_chain_f32(C.byref(d), C.byref(g), None))
        assert g.value == g2n
        gave_up, misplaced = C.c_int(-1), C.c_int(-1)
        et.check(lib.et_device_sync())
        et.check(lib.et_encoder_chain_status(sync.ptr, C.byref(gave_up), C.byref(misplaced)))
        assert (gave_up.value, misplaced.value) == (0, 0)
        for k in ("V1", "fin1", "Hh", "V2", "fin2", "QKV"):
            x, y = a[k].numpy(), b[k].numpy()
            assert np.array_equal(x.view(np.uint8), y.view(np.uint8)), k
        assert np.array_equal(a["st1"].numpy()[:g1n], b["st1"].numpy()[:g1n])
        assert np.array_equal(a["st2"].numpy()[:g2n], b["st2"].numpy()[:g2n])
        # and against the mathematics (loosely: the pieces are checked one by one above)
        v1 = L.linear(Hn.f32(z.numpy()), Hn.f32(wo.dense), Hn.f32(wo.bias)).numpy() + resid.numpy()
        assert Hn.max_abs(b["V1"].numpy(), v1) <= 1e-4 * max(1.0, float(np.abs(v1).max()))
        # a description whose widths do not chain is refused
        d.down = pu.value
        assert lib.et_encoder_chain_supported(C.byref(d)) == 0
        assert lib.et_encoder_chain_f32(C.byref(d), C.byref(g), None) == et.ET_ERR_UNSUPPORTED
    finally:
        et.check(lib.et_device_sync())
        for h in (po, pu, pd, pq):
            et.check(lib.et_bsr16_pack_destroy(h))
