"""binary32 twins on the GPU against the CPU oracle, and the dense fp32 encoder layer of the
first benchmark configuration (one BERT-base layer, batch 1, seq 128) composed from them,
to the fp32-path tolerance max-abs 1e-4."""
import ctypes as C
import importlib.util
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import layers as L
from tests import harness as Hn

pytestmark = pytest.mark.gpu
up = Hn.up
GOLDEN = Path(__file__).parent / "golden"
TOL_F32 = 1e-4
ACT = {0: None, 1: "relu", 2: "gelu"}


def randf(shape, seed, std=1.0):
    return (torch.randn(*shape, generator=Hn.rng(seed)) * std).numpy().astype(np.float32)


@pytest.mark.parametrize("T,inp,out,act", [(128, 768, 2304, 0), (128, 768, 3072, 2), (128, 3072, 768, 0),
                                           (100, 48, 20, 1), (1, 16, 4, 0), (77, 160, 132, 2)])
def test_linear_dense_f32(et, T, inp, out, act):
    W, b, x = randf((out, inp), 1, 0.05), randf((out,), 2, 0.1), randf((T, inp), 3)
    d_y = et.DeviceBuffer.empty((T, out), np.float32)
    et.check(et.lib().et_linear_dense_f32(up(et, W).ptr, up(et, b).ptr, up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    want = torch.from_numpy(x.astype(np.float64) @ W.astype(np.float64).T + b)  # binary64 reference
    want = L.ACTS[ACT[act]](want).numpy()
    # fp32 accumulation of `inp` products, |y| up to ~10: error ~ sqrt(inp) * 6e-8 * |y|
    assert Hn.max_abs(d_y.numpy(), want) <= 5e-5


def test_linear_dense_f32_no_bias_and_bad_args(et):
    W, x = randf((32, 32), 4), randf((16, 32), 5)
    d_y = et.DeviceBuffer.empty((16, 32), np.float32)
    et.check(et.lib().et_linear_dense_f32(up(et, W).ptr, None, up(et, x).ptr, d_y.ptr, 16, 32, 32, 0, None))
    assert Hn.max_abs(d_y.numpy(), x @ W.T) <= 1e-5
    assert et.lib().et_linear_dense_f32(up(et, W).ptr, None, up(et, x).ptr, d_y.ptr, 16, 24, 32, 0, None) \
        == et.ET_ERR_UNSUPPORTED
    assert et.lib().et_linear_dense_f32(None, None, up(et, x).ptr, d_y.ptr, 16, 32, 32, 0, None) == et.ET_ERR_INVALID_ARG


@pytest.mark.parametrize("B,S,nh,hd,causal,lens,mask", [
    (1, 128, 12, 64, False, None, False), (3, 128, 12, 64, False, [128, 64, 97], False),
    (2, 64, 4, 32, True, None, False), (2, 48, 2, 128, False, [0, 48], True), (1, 512, 2, 64, True, [300], False),
    (2, 64, 3, 48, False, [64, 20], False), (1, 32, 2, 16, True, None, False)])
def test_mha_fused_f32(et, B, S, nh, hd, causal, lens, mask):
    H = nh * hd
    qkv = randf((B * S, 3 * H), 6)
    d_qkv = up(et, qkv)
    d_z = et.DeviceBuffer.empty((B * S, H), np.float32)
    m = randf((S, S), 7) if mask else None
    if mask:
        m[:, 5] = -np.inf
    d_m = up(et, m) if mask else None
    d_l = up(et, np.asarray(lens, np.int32)) if lens is not None else None
    et.check(et.lib().et_mha_fused_f32(d_qkv.ptr, d_qkv.offset(4 * H), d_qkv.offset(8 * H), 3 * H, 3 * H, 3 * H,
                                       d_z.ptr, H, d_m.ptr if mask else None, d_l.ptr if lens is not None else None,
                                       B, S, nh, hd, hd ** -0.5, et.MHA_CAUSAL if causal else 0, None))
    t = torch.from_numpy(qkv)
    want = L.mha(t[:, :H], t[:, H:2 * H], t[:, 2 * H:], nh, B, mask=torch.from_numpy(m) if mask else None,
                 lens=lens, causal=causal)
    assert Hn.max_abs(d_z.numpy(), want.numpy()) <= 1e-5


@pytest.mark.parametrize("rows,H", [(128, 768), (33, 1024), (5, 4100), (7, 64)])
def test_layernorm_f32(et, rows, H):
    src, skip = randf((rows, H), 8, 2.0), randf((rows, H), 9)
    gamma, beta = 1 + randf((H,), 10, 0.1), randf((H,), 11, 0.1)
    d_out = et.DeviceBuffer.empty((rows, H), np.float32)
    et.check(et.lib().et_skip_layernorm_f32(d_out.ptr, up(et, src).ptr, up(et, skip).ptr, up(et, gamma).ptr,
                                            up(et, beta).ptr, rows, H, 1e-5, None))
    want = torch.nn.functional.layer_norm(torch.from_numpy(src + skip).double(), (H,), torch.from_numpy(gamma).double(),
                                          torch.from_numpy(beta).double(), 1e-5).float().numpy()
    assert Hn.max_abs(d_out.numpy(), want) <= 1e-5
    et.check(et.lib().et_layernorm_f32(d_out.ptr, up(et, src).ptr, up(et, gamma).ptr, up(et, beta).ptr, rows, H,
                                       1e-5, None))
    want = torch.nn.functional.layer_norm(torch.from_numpy(src).double(), (H,), torch.from_numpy(gamma).double(),
                                          torch.from_numpy(beta).double(), 1e-5).float().numpy()
    assert Hn.max_abs(d_out.numpy(), want) <= 1e-5


def test_gelu_relu_f32(et):
    x = randf((100003,), 12, 3.0)
    d_o = et.DeviceBuffer.empty(x.shape, np.float32)
    et.check(et.lib().et_gelu_f32(d_o.ptr, up(et, x).ptr, x.size, None))
    want = torch.nn.functional.gelu(torch.from_numpy(x).double(), approximate="tanh").float().numpy()
    assert Hn.max_abs(d_o.numpy(), want) <= 2e-6
    et.check(et.lib().et_relu_f32(d_o.ptr, up(et, x).ptr, x.size, None))
    assert np.array_equal(d_o.numpy(), np.maximum(x, 0))


def f32_layer(et, x, p, nh, B, act=2, lens=None):
    """One post-LN encoder layer from the binary32 entry points (weights: dict of numpy fp32)."""
    lib = et.lib()
    T, H = x.shape
    FF = p["W1"].shape[0]
    S = T // B
    f = lambda shape: et.DeviceBuffer.empty(shape, np.float32)
    d = {k: up(et, np.ascontiguousarray(v, dtype=np.float32)) for k, v in p.items()}
    d_x, qkv, z, a, y1, ff, f2, out = up(et, x), f((T, 3 * H)), f((T, H)), f((T, H)), f((T, H)), f((T, FF)), \
        f((T, H)), f((T, H))
    d_l = up(et, np.asarray(lens, np.int32)) if lens is not None else None
    et.check(lib.et_linear_dense_f32(d["Wqkv"].ptr, d["bqkv"].ptr, d_x.ptr, qkv.ptr, T, H, 3 * H, 0, None))
    et.check(lib.et_mha_fused_f32(qkv.ptr, qkv.offset(4 * H), qkv.offset(8 * H), 3 * H, 3 * H, 3 * H, z.ptr, H, None,
                                  d_l.ptr if d_l else None, B, S, nh, H // nh, (H // nh) ** -0.5, 0, None))
    et.check(lib.et_linear_dense_f32(d["Wo"].ptr, d["bo"].ptr, z.ptr, a.ptr, T, H, H, 0, None))
    et.check(lib.et_skip_layernorm_f32(y1.ptr, a.ptr, d_x.ptr, d["g1"].ptr, d["be1"].ptr, T, H, 1e-5, None))
    et.check(lib.et_linear_dense_f32(d["W1"].ptr, d["b1"].ptr, y1.ptr, ff.ptr, T, H, FF, act, None))
    et.check(lib.et_linear_dense_f32(d["W2"].ptr, d["b2"].ptr, ff.ptr, f2.ptr, T, FF, H, 0, None))
    et.check(lib.et_skip_layernorm_f32(out.ptr, f2.ptr, y1.ptr, d["g2"].ptr, d["be2"].ptr, T, H, 1e-5, None))
    return out.numpy()


def test_dense_fp32_encoder_layer_matches_library_fixture_and_oracle(et):
    """First benchmark configuration: one dense BERT-base layer, fp32, batch 1, seq 128, N(0, 0.02)
    weights, zero biases, unit LayerNorm, N(0, 1) input.  Checked against the committed output of
    torch.nn.TransformerEncoderLayer and against the CPU oracle, both to max-abs 1e-4."""
    spec = importlib.util.spec_from_file_location("mk", GOLDEN / "make_encoder_layer_c1.py")
    mk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mk)
    sp = mk.seeded_params()
    H, FF = mk.H, mk.FF
    z = lambda n: np.zeros(n, np.float32)
    p = {"Wqkv": sp["Wqkv"].numpy(), "bqkv": z(3 * H), "Wo": sp["Wo"].numpy(), "bo": z(H), "W1": sp["W1"].numpy(),
         "b1": z(FF), "W2": sp["W2"].numpy(), "b2": z(H), "g1": np.ones(H, np.float32), "be1": z(H),
         "g2": np.ones(H, np.float32), "be2": z(H)}
    y = f32_layer(et, sp["x"].numpy(), p, mk.NH, 1)
    fx = np.load(GOLDEN / "encoder_layer_c1.npz")
    assert np.max(np.abs(y[:8] - fx["y_head"])) <= TOL_F32
    assert abs(float(y.astype(np.float64).sum()) - float(fx["y_sum"])) <= 1e-2
    assert abs(float(np.abs(y.astype(np.float64)).sum()) - float(fx["y_abs_sum"])) <= 1e-1
    P = L.LayerParams(sp["Wqkv"], torch.zeros(3 * H), sp["Wo"], torch.zeros(H), sp["W1"], torch.zeros(FF), sp["W2"],
                      torch.zeros(H), torch.ones(H), torch.zeros(H), torch.ones(H), torch.zeros(H))
    want = L.encoder_layer(sp["x"], P, L.LayerConfig(nh=mk.NH, act="gelu", eps=1e-5)).numpy()
    err = float(np.max(np.abs(y - want)))
    print(f"dense fp32 layer max-abs vs oracle: {err:.2e}")
    assert err <= TOL_F32


def test_fp32_layer_with_biases_padding_and_batch(et):
    H, nh, FF, S, B = 256, 4, 512, 64, 3
    g = lambda shape, seed, std: randf(shape, seed, std)
    p = {"Wqkv": g((3 * H, H), 20, 0.05), "bqkv": g((3 * H,), 21, 0.1), "Wo": g((H, H), 22, 0.05), "bo": g((H,), 23, 0.1),
         "W1": g((FF, H), 24, 0.05), "b1": g((FF,), 25, 0.1), "W2": g((H, FF), 26, 0.05), "b2": g((H,), 27, 0.1),
         "g1": 1 + g((H,), 28, 0.1), "be1": g((H,), 29, 0.1), "g2": 1 + g((H,), 30, 0.1), "be2": g((H,), 31, 0.1)}
    x = randf((B * S, H), 32)
    lens = [64, 16, 33]
    y = f32_layer(et, x, p, nh, B, act=1, lens=lens)
    t = {k: torch.from_numpy(v) for k, v in p.items()}
    P = L.LayerParams(t["Wqkv"], t["bqkv"], t["Wo"], t["bo"], t["W1"], t["b1"], t["W2"], t["b2"], t["g1"], t["be1"],
                      t["g2"], t["be2"])
    want = L.encoder_layer(torch.from_numpy(x), P, L.LayerConfig(nh=nh, B=B, act="relu", lens=lens)).numpy()
    assert Hn.max_abs(y, want) <= TOL_F32


# ---- binary32 twins over the sparse weight containers ---------------------------------------
# Each is checked against the binary64 product with the dense image the format oracle builds
# from the same structure arrays (oracle/formats.py), to the accumulation error of `inp` binary32
# products.
def _want64(x, Wd, b, act):
    y = torch.from_numpy(x.astype(np.float64) @ Wd.astype(np.float64).T + (0 if b is None else b.astype(np.float64)))
    return L.ACTS[ACT[act]](y).numpy()


@pytest.mark.parametrize("T,inp,out,sp,act", [(128, 768, 2304, 0.8, 0), (1024, 768, 3072, 0.8, 2),
                                              (2048, 3072, 768, 0.9, 0), (100, 48, 32, 0.5, 1), (1, 16, 16, 0.0, 0),
                                              (77, 160, 144, 0.95, 2)])
def test_linear_bsr16_f32(et, T, inp, out, sp, act):
    from oracle import formats as F
    row_ptr, col_idx = F.gen_tile_pattern(out, inp, sp, seed=31)
    tiles = randf((max(len(col_idx), 1), 256), 32, 0.05)
    Wd = F.bsr16_to_dense(row_ptr, col_idx, tiles[:len(col_idx)], inp)
    b, x = randf((out,), 33, 0.1), randf((T, inp), 34)
    d_y = et.DeviceBuffer.empty((T, out), np.float32)
    ci = col_idx if len(col_idx) else np.zeros(1, np.int32)
    et.check(et.lib().et_linear_bsr16_f32(up(et, row_ptr).ptr, up(et, ci).ptr, up(et, tiles).ptr, up(et, b).ptr,
                                          up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    assert Hn.max_abs(d_y.numpy(), _want64(x, Wd, b, act)) <= 5e-5


def test_linear_bsr16_f32_closed_form_and_bad_args(et):
    """All-ones tiles and inputs: every output is 16 x (tiles of its block-row) + bias, exactly."""
    from oracle import formats as F
    T, inp, out = 48, 256, 64
    row_ptr, col_idx = F.gen_tile_pattern(out, inp, 0.6, seed=5)
    tiles = np.ones((len(col_idx), 256), np.float32)
    b = np.arange(out, dtype=np.float32)
    d_y = et.DeviceBuffer.empty((T, out), np.float32)
    args = (up(et, row_ptr).ptr, up(et, col_idx).ptr, up(et, tiles).ptr, up(et, b).ptr,
            up(et, np.ones((T, inp), np.float32)).ptr, d_y.ptr)
    et.check(et.lib().et_linear_bsr16_f32(*args, T, inp, out, 0, None))
    want = np.repeat(16.0 * np.diff(row_ptr), 16)[None, :] + b[None, :]
    assert np.array_equal(d_y.numpy(), np.broadcast_to(want, (T, out)).astype(np.float32))
    assert et.lib().et_linear_bsr16_f32(*args, T, inp, 60, 0, None) == et.ET_ERR_UNSUPPORTED
    assert et.lib().et_linear_bsr16_f32(*args, T, inp, out, 7, None) == et.ET_ERR_INVALID_ARG
    assert et.lib().et_linear_bsr16_f32(None, *args[1:], T, inp, out, 0, None) == et.ET_ERR_INVALID_ARG


@pytest.mark.parametrize("T,inp,out,sp,act", [(2048, 768, 768, 0.5, 0), (128, 768, 3072, 0.5, 2), (100, 48, 64, 0.3, 1),
                                              (7, 3072, 768, 0.9, 0)])
def test_linear_rowpruned_f32(et, T, inp, out, sp, act):
    from oracle import formats as F
    row_id = F.gen_row_ids(out, sp, seed=8)
    rows, b, x = randf((len(row_id), inp), 35, 0.05), randf((out,), 36, 0.1), randf((T, inp), 37)
    d_y = et.DeviceBuffer.from_numpy(np.full((T, out), np.nan, np.float32))  # every element must be written
    et.check(et.lib().et_linear_rowpruned_f32(up(et, rows).ptr, up(et, row_id).ptr, len(row_id), up(et, b).ptr,
                                              up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    got = d_y.numpy()
    assert Hn.max_abs(got, _want64(x, F.row_mat_to_dense(rows, row_id, out), b, act)) <= 5e-5
    dead = np.setdiff1d(np.arange(out), row_id)
    bias_only = L.ACTS[ACT[act]](torch.from_numpy(b).double()).numpy()
    assert Hn.max_abs(got[:, dead], np.broadcast_to(bias_only[dead], (T, len(dead)))) <= 1e-6
    d_c = et.DeviceBuffer.empty((T, len(row_id)), np.float32)
    et.check(et.lib().et_linear_rowpruned_compact_f32(up(et, rows).ptr, up(et, row_id).ptr, len(row_id),
                                                      up(et, b).ptr, up(et, x).ptr, d_c.ptr, T, inp, None))
    assert Hn.max_abs(d_c.numpy(), _want64(x, rows, b[row_id], 0)) <= 5e-5
    et.check(et.lib().et_linear_rowpruned_compact_f32(up(et, rows).ptr, up(et, row_id).ptr, len(row_id),
                                                      None, up(et, x).ptr, d_c.ptr, T, inp, None))
    assert Hn.max_abs(d_c.numpy(), _want64(x, rows, None, 0)) <= 5e-5


@pytest.mark.parametrize("T,inp,out,sp,act", [(2048, 768, 768, 0.5, 0), (128, 768, 3072, 0.5, 2), (33, 160, 48, 0.3, 1),
                                              (128, 3072, 768, 0.9, 0)])
def test_linear_colpruned_f32(et, T, inp, out, sp, act):
    from oracle import formats as F
    col_id = F.gen_col_ids(inp, sp, seed=12)  # unsorted, as the reference generator leaves them
    cols, b, x = randf((out, len(col_id)), 38, 0.05), randf((out,), 39, 0.1), randf((T, inp), 40)
    d_y = et.DeviceBuffer.empty((T, out), np.float32)
    et.check(et.lib().et_linear_colpruned_f32(up(et, cols).ptr, up(et, col_id).ptr, len(col_id), up(et, b).ptr,
                                              up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    assert Hn.max_abs(d_y.numpy(), _want64(x, F.col_mat_to_dense(cols, col_id, inp), b, act)) <= 5e-5


@pytest.mark.parametrize("T,inp,out,sp,act", [(2048, 768, 768, 0.8, 0), (128, 768, 3072, 0.5, 2), (16, 32, 16, 0.0, 0),
                                              (81, 3072, 64, 0.9, 1)])
def test_linear_vec1x16_f32(et, T, inp, out, sp, act):
    from oracle import formats as F
    keep = np.repeat(torch.rand(out, inp // 16, generator=Hn.rng(16)).numpy() >= sp, 16, axis=1)
    W = randf((out, inp), 41, 0.05) * keep
    tile_idx, row_idx, data = F.dense_to_1x16(W)
    data = np.ascontiguousarray(data, np.float32)
    assert np.array_equal(F.mat1x16_to_dense(tile_idx, row_idx, data, out, inp), W)
    b, x = randf((out,), 42, 0.1), randf((T, inp), 43)
    d_y = et.DeviceBuffer.empty((T, out), np.float32)
    row_idx_d = row_idx if len(row_idx) else np.zeros(1, np.int32)
    data_d = data if data.size else np.zeros((16, 16), np.float32)
    et.check(et.lib().et_linear_vec1x16_f32(up(et, tile_idx).ptr, up(et, row_idx_d).ptr, up(et, data_d).ptr,
                                            up(et, b).ptr, up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    assert Hn.max_abs(d_y.numpy(), _want64(x, W, b, act)) <= 5e-5


def test_linear_vec1x16_f32_unsorted_rows_in_a_cell(et):
    from oracle import formats as F
    T, inp, out = 32, 64, 32
    tile_idx, row_idx = F.gen_1x16_pattern(out, inp, 0.5, seed=3)  # keeps the permuted order inside a cell
    data = randf((((len(row_idx) + 15) // 16) * 16, 16), 44, 0.1)
    W = F.mat1x16_to_dense(tile_idx, row_idx, data, out, inp)
    x = randf((T, inp), 45)
    d_y = et.DeviceBuffer.empty((T, out), np.float32)
    et.check(et.lib().et_linear_vec1x16_f32(up(et, tile_idx).ptr, up(et, row_idx).ptr, up(et, data).ptr, None,
                                            up(et, x).ptr, d_y.ptr, T, inp, out, 0, None))
    assert Hn.max_abs(d_y.numpy(), _want64(x, W, None, 0)) <= 1e-5


@pytest.mark.parametrize("T,inp,out,sp,act", [(1024, 768, 768, 0.9, 0), (100, 768, 3072, 0.95, 2), (7, 40, 12, 0.5, 1),
                                              (64, 40000, 16, 0.999, 0)])
def test_linear_csr_f32(et, T, inp, out, sp, act):
    from oracle import formats as F
    mask = torch.rand(out, inp, generator=Hn.rng(22)).numpy() >= sp
    W = randf((out, inp), 46, 0.05) * mask
    indptr, indices, data = F.dense_to_csr(W)
    data = np.ascontiguousarray(data, np.float32)
    b, x = randf((out,), 47, 0.1), randf((T, inp), 48)
    d_y = et.DeviceBuffer.from_numpy(np.full((T, out), np.nan, np.float32))
    et.check(et.lib().et_linear_csr_f32(up(et, indptr).ptr, up(et, indices).ptr,
                                        up(et, data if data.size else np.zeros(1, np.float32)).ptr,
                                        up(et, b).ptr, up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    assert Hn.max_abs(d_y.numpy(), _want64(x, W, b, act)) <= 5e-5


def test_linear_csr_f32_reference_fixture(et):
    """The reference's dense_4_3.csr (all ones): y = sum of the 3 inputs + bias."""
    from oracle import formats as F
    nrow, ncol, nnz, indptr, indices, data = F.read_csr(str(GOLDEN / "dense_4_3.csr"))
    x = randf((5, ncol), 49)
    b = np.array([0.5, -1, 2, 0], np.float32)
    d_y = et.DeviceBuffer.empty((5, nrow), np.float32)
    et.check(et.lib().et_linear_csr_f32(up(et, indptr).ptr, up(et, indices).ptr, up(et, data.astype(np.float32)).ptr,
                                        up(et, b).ptr, up(et, x).ptr, d_y.ptr, 5, ncol, nrow, 0, None))
    assert Hn.max_abs(d_y.numpy(), x.astype(np.float64).sum(1, keepdims=True) + b) <= 1e-6


def test_tile_sparse_fp32_encoder_stack(et):
    """The benchmark's pruned encoder (BERT-base, 80 % 16x16 tile sparsity on Q/K/V/O and both FFN matrices, batch 8
    of 128 tokens with right padding) composed from the binary32 entry points alone, three layers deep: tile-sparse
    Linear, fused attention, SkipLayerNorm.  Against the oracle's binary32 forward, max-abs 2e-4."""
    from oracle import formats as F
    lib = et.lib()
    H, nh, FF, S, B, depth = 768, 12, 3072, 128, 8, 3
    T = B * S
    lens = [128, 100, 64, 128, 17, 96, 128, 80]
    d_l = up(et, np.asarray(lens, np.int32))
    f = lambda shape: et.DeviceBuffer.empty(shape, np.float32)
    qkv, z, a, y1, ff, f2 = f((T, 3 * H)), f((T, H)), f((T, H)), f((T, H)), f((T, FF)), f((T, H))

    def sparse(out, inp, seed):
        row_ptr, col_idx = F.gen_tile_pattern(out, inp, 0.8, seed=seed)
        tiles = randf((len(col_idx), 256), seed + 1, 0.03)
        b = randf((out,), seed + 2, 0.05)
        dev = (up(et, row_ptr), up(et, col_idx), up(et, tiles), up(et, b))
        return dev, torch.from_numpy(F.bsr16_to_dense(row_ptr, col_idx, tiles, inp)), torch.from_numpy(b)

    x = randf((T, H), 900)
    cur, want = up(et, x), torch.from_numpy(x)
    for layer in range(depth):
        s0 = 1000 + 50 * layer
        (dq, Wq, bq), (do, Wo, bo) = sparse(3 * H, H, s0), sparse(H, H, s0 + 10)
        (d1, W1, b1), (d2, W2, b2) = sparse(FF, H, s0 + 20), sparse(H, FF, s0 + 30)
        g1, be1, g2, be2 = 1 + randf((H,), s0 + 40, 0.1), randf((H,), s0 + 41, 0.1), 1 + randf((H,), s0 + 42, 0.1), \
            randf((H,), s0 + 43, 0.1)
        dg1, dbe1, dg2, dbe2 = up(et, g1), up(et, be1), up(et, g2), up(et, be2)
        lin = lambda w, src, dst, n_in, n_out, act: et.check(lib.et_linear_bsr16_f32(
            w[0].ptr, w[1].ptr, w[2].ptr, w[3].ptr, src.ptr, dst.ptr, T, n_in, n_out, act, None))
        out = f((T, H))
        lin(dq, cur, qkv, H, 3 * H, 0)
        et.check(lib.et_mha_fused_f32(qkv.ptr, qkv.offset(4 * H), qkv.offset(8 * H), 3 * H, 3 * H, 3 * H, z.ptr, H, None,
                                      d_l.ptr, B, S, nh, H // nh, (H // nh) ** -0.5, 0, None))
        lin(do, z, a, H, H, 0)
        et.check(lib.et_skip_layernorm_f32(y1.ptr, a.ptr, cur.ptr, dg1.ptr, dbe1.ptr, T, H, 1e-5, None))
        lin(d1, y1, ff, H, FF, 2)
        lin(d2, ff, f2, FF, H, 0)
        et.check(lib.et_skip_layernorm_f32(out.ptr, f2.ptr, y1.ptr, dg2.ptr, dbe2.ptr, T, H, 1e-5, None))
        cur = out
        t = torch.from_numpy
        P = L.LayerParams(Wq, bq, Wo, bo, W1, b1, W2, b2, t(g1), t(be1), t(g2), t(be2))
        want = L.encoder_layer(want, P, L.LayerConfig(nh=nh, B=B, act="gelu", lens=lens))
    got, want = cur.numpy(), want.numpy()
    for b in range(B):  # rows past a sequence's length are padding: not compared
        got[b * S + lens[b]:(b + 1) * S] = 0
        want[b * S + lens[b]:(b + 1) * S] = 0
    err = Hn.max_abs(got, want)
    print(f"tile-sparse fp32 stack, {depth} layers: max-abs vs oracle {err:.2e}")
    assert err <= 2e-4


def _f32_model(et, H, nh, FF, S, B, nlayer, act, use_graph, causal=False):
    desc = et.ModelDesc(H, H, S, nh, FF, H, nlayer, B, act, 1e-5, int(causal), int(use_graph), 0)
    h = C.c_void_p()
    et.check(et.lib().et_model_f32_create(C.byref(desc), C.byref(h)))
    return h


def _np(a):
    return np.ascontiguousarray(a).ctypes.data


@pytest.mark.parametrize("use_graph", [True, False])
def test_fp32_model_handle_tile_sparse_stack(et, use_graph):
    """et_model_f32_*: three pruned layers (80 % tiles; the last layer's FFN dense), batch 4 of 64 tokens with right
    padding, GELU, against the oracle's binary32 forward; a second forward on the same buffers replays the graph."""
    from oracle import formats as F
    lib = et.lib()
    H, nh, FF, S, B, depth = 256, 4, 512, 64, 4, 3
    T = B * S
    lens = np.array([64, 20, 33, 48], np.int32)
    h = _f32_model(et, H, nh, FF, S, B, depth, et.ACT_GELU, use_graph)
    want = torch.from_numpy(randf((T, H), 700))
    x = want.numpy().copy()
    shapes = {0: (3 * H, H), 1: (H, H), 2: (FF, H), 3: (H, FF)}
    params = []
    for layer in range(depth):
        mats = []
        for which, (out, inp) in shapes.items():
            seed = 800 + 40 * layer + 7 * which
            b = randf((out,), seed + 2, 0.05)
            if layer == depth - 1 and which >= 2:  # dense
                W = randf((out, inp), seed, 0.05)
                et.check(lib.et_model_f32_set_dense(h, layer, which, _np(W), _np(b)))
            else:
                row_ptr, col_idx = F.gen_tile_pattern(out, inp, 0.8, seed=seed)
                tiles = randf((len(col_idx), 256), seed + 1, 0.05)
                W = F.bsr16_to_dense(row_ptr, col_idx, tiles, inp)
                et.check(lib.et_model_f32_set_bsr16(h, layer, which, _np(row_ptr), _np(col_idx), _np(tiles), len(col_idx),
                                                    _np(b)))
            mats += [torch.from_numpy(W), torch.from_numpy(b)]
        norms = []
        for which in range(2):
            g, be = 1 + randf((H,), 900 + 10 * layer + which, 0.1), randf((H,), 950 + 10 * layer + which, 0.1)
            et.check(lib.et_model_f32_set_norm(h, layer, which, _np(g), _np(be)))
            norms += [torch.from_numpy(g), torch.from_numpy(be)]
        params.append(L.LayerParams(*mats, *norms))
    et.check(lib.et_model_f32_set_lens(h, _np(lens)))
    et.check(lib.et_model_f32_finalize(h))
    assert lib.et_model_f32_set_norm(h, 0, 0, _np(x), _np(x)) == et.ET_ERR_INVALID_ARG  # frozen after finalize
    d_x, d_y = up(et, x), et.DeviceBuffer.empty((T, H), np.float32)
    for p in params:
        want = L.encoder_layer(want, p, L.LayerConfig(nh=nh, B=B, act="gelu", lens=lens.tolist()))
    want = want.numpy()
    for rep in range(2):
        nan = np.full((T, H), np.nan, np.float32)
        et.check(lib.et_memcpy_h2d(d_y.ptr, _np(nan), nan.nbytes))
        et.check(lib.et_model_f32_forward(h, d_y.ptr, d_x.ptr, None))
        et.check(lib.et_model_f32_sync(h))
        got = d_y.numpy()
        for b in range(B):  # rows past a sequence's length are padding: not compared
            got[b * S + lens[b]:(b + 1) * S] = 0
            want[b * S + lens[b]:(b + 1) * S] = 0
        err = Hn.max_abs(got, want)
        print(f"fp32 model handle (graph={use_graph}) pass {rep}: max-abs vs oracle {err:.2e}")
        assert err <= TOL_F32
    et.check(lib.et_model_f32_destroy(h))


def test_fp32_model_handle_rejects_bad_use(et):
    lib = et.lib()
    h = C.c_void_p()
    bad = et.ModelDesc(256, 128, 64, 4, 512, 256, 1, 1, et.ACT_GELU, 1e-5, 0, 0, 0)  # kdim != vdim
    assert lib.et_model_f32_create(C.byref(bad), C.byref(h)) == et.ET_ERR_INVALID_ARG
    h = _f32_model(et, 64, 4, 128, 16, 1, 1, et.ACT_RELU, False)
    assert lib.et_model_f32_finalize(h) == et.ET_ERR_INVALID_ARG  # weights never set
    W = randf((192, 64), 1, 0.05)
    assert lib.et_model_f32_set_dense(h, 1, 0, _np(W), None) == et.ET_ERR_INVALID_ARG  # layer out of range
    assert lib.et_model_f32_set_dense(h, 0, 4, _np(W), None) == et.ET_ERR_INVALID_ARG  # bad selector
    rp = np.zeros(13, np.int32)
    rp[1:] = 1
    assert lib.et_model_f32_set_bsr16(h, 0, 0, _np(rp), _np(np.array([9], np.int32)), _np(randf((1, 256), 2)), 1,
                                      None) != et.ET_OK  # column tile outside the matrix
    x = np.zeros((16, 64), np.float32)
    assert lib.et_model_f32_forward(h, _np(x), _np(x), None) == et.ET_ERR_INVALID_ARG  # not finalized
    et.check(lib.et_model_f32_destroy(h))
