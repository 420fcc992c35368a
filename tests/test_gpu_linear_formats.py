"""GPU parity of the dense / row-pruned / column-pruned / 1x16 / CSR Linear kernels and the
GEMM behind them against the CPU oracle (same seeded inputs, fp16 storage, fp32 accumulation)."""
import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import layers as L
from tests import harness as Hn

pytestmark = pytest.mark.gpu
ACT = {0: None, 1: "relu", 2: "gelu"}


up = Hn.up


@pytest.mark.parametrize("T,inp,out,act", [(2048, 768, 768, 0), (1024, 768, 3072, 2), (128, 3072, 768, 0),
                                           (16, 16, 16, 1), (48, 80, 112, 0), (2048, 1024, 1024, 0),
                                           # one shape per tile of the direct-to-LDS kernel: 256x256, 128x128,
                                           # 128x64, 64x64 with three LDS buffers, a single K stage
                                           (4096, 192, 4096, 2), (2048, 128, 4096, 1), (2048, 192, 2304, 0),
                                           # 256x256 tiles with a single K stage, and with many
                                           (4096, 64, 4096, 0), (4096, 1024, 4096, 1),
                                           (512, 1536, 768, 2), (256, 64, 256, 0),
                                           # edges that are multiples of 16 only (clamped loads, zeroed K tail,
                                           # masked stores): 16, 32 and 48 k-values in the last stage
                                           (1008, 720, 400, 2), (80, 96, 2064, 1), (2032, 176, 48, 0),
                                           # few 64x64 tiles and a long K: one 16x16 tile per workgroup, K split over
                                           # its waves (K a multiple of 32, of 16 only, more than one round of loads)
                                           (128, 768, 768, 2), (16, 272, 16, 0), (128, 3072, 80, 1), (32, 6160, 48, 0),
                                           # the largest results that kernel takes: 2048 tiles of 16 x 16
                                           (512, 768, 1024, 2), (128, 768, 2304, 0), (448, 784, 720, 1),
                                           # edges of 16 with enough work for the 128 x 64 and 128 x 128 tiles
                                           (2048, 768, 2928, 2), (2000, 720, 2096, 1), (4080, 208, 4112, 0), (8176, 80, 8208, 1)])
def test_linear_dense(et, T, inp, out, act):
    W, b, x = Hn.randn((out, inp), 1, 0.02), Hn.randn((out,), 2, 0.1), Hn.randn((T, inp), 3)
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.linear_dense(up(et, W), up(et, b), up(et, x), d_y, T, inp, out, act)
    want = L.linear(Hn.f32(x), Hn.f32(W), Hn.f32(b), ACT[act], torch.float16).numpy()
    assert Hn.max_abs(d_y.numpy(), want) <= 4e-3


def _random_dense_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        big = rng.random() < 0.3  # some shapes large enough for the 128- and 256-wide tiles
        T = 16 * int(rng.integers(1, 200 if big else 40))
        inp = 16 * int(rng.integers(1, 100))
        out = 16 * int(rng.integers(1, 200 if big else 60))
        cases.append((T, inp, out, int(rng.integers(0, 3)), int(rng.integers(1, 1 << 30))))
    return cases


@pytest.mark.parametrize("T,inp,out,act,seed", _random_dense_cases(32, 20211117))
def test_linear_dense_random_shapes(et, T, inp, out, act, seed):
    """Seeded random shapes, multiples of 16 only: whichever GEMM form and tile the shape picks (one 16x16 tile per
    workgroup, 64x64, the direct-to-LDS tiles, full or ragged edges), and the row- and column-pruned Linears on
    top of the same GEMM with a random half of the features."""
    W, b, x = Hn.randn((out, inp), seed & 0xFFFF, 0.02), Hn.randn((out,), 2, 0.1), Hn.randn((T, inp), 3)
    d_W, d_b, d_x = up(et, W), up(et, b), up(et, x)
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.linear_dense(d_W, d_b, d_x, d_y, T, inp, out, act)
    want = L.linear(Hn.f32(x), Hn.f32(W), Hn.f32(b), ACT[act], torch.float16).numpy()
    assert Hn.max_abs(d_y.numpy(), want) <= 4e-3
    lib = et.lib()
    row_id = F.gen_row_ids(out, 0.5, seed=seed)
    if len(row_id):
        rows = np.ascontiguousarray(W[row_id])
        et.check(lib.et_fill_f16(d_y.ptr, T * out, 0x7E00, None))
        et.check(lib.et_linear_rowpruned_f16(up(et, rows).ptr, up(et, row_id).ptr, len(row_id), d_b.ptr, d_x.ptr,
                                             d_y.ptr, T, inp, out, act, None))
        want_r = L.linear_rowpruned(Hn.f32(x), Hn.f32(rows), row_id, out, Hn.f32(b), ACT[act], torch.float16).numpy()
        assert Hn.max_abs(d_y.numpy(), want_r) <= 4e-3
    col_id = F.gen_col_ids(inp, 0.5, seed=seed + 1)
    if len(col_id):
        cols = np.ascontiguousarray(W[:, col_id])
        et.check(lib.et_fill_f16(d_y.ptr, T * out, 0x7E00, None))
        et.check(lib.et_linear_colpruned_f16(up(et, cols).ptr, up(et, col_id).ptr, len(col_id), d_b.ptr, d_x.ptr,
                                             d_y.ptr, T, inp, out, act, None))
        want_c = L.linear_colpruned(Hn.f32(x), Hn.f32(cols), col_id, Hn.f32(b), ACT[act], torch.float16).numpy()
        assert Hn.max_abs(d_y.numpy(), want_c) <= 4e-3


@pytest.mark.parametrize("T,inp,out", [(4096, 128, 4096), (512, 768, 768)])
def test_linear_dense_without_bias(et, T, inp, out):
    W, x = Hn.randn((out, inp), 21, 0.02), Hn.randn((T, inp), 22)
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.check(et.lib().et_linear_dense_f16(up(et, W).ptr, None, up(et, x).ptr, d_y.ptr, T, inp, out, 0, None))
    want = L.linear(Hn.f32(x), Hn.f32(W), None, None, torch.float16).numpy()
    assert Hn.max_abs(d_y.numpy(), want) <= 4e-3


def test_linear_dense_closed_form_ones(et):
    """All-ones weights and input, bias 0.5: every output is in_size + 0.5 (the closed form of the
    reference driver, Linear/test/test_cublas.cu:12-19, at a width whose sum fp16 represents)."""
    T, inp, out = 64, 256, 128
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.linear_dense(up(et, np.ones((out, inp), np.float16)), up(et, np.full(out, 0.5, np.float16)),
                    up(et, np.ones((T, inp), np.float16)), d_y, T, inp, out)
    assert np.all(d_y.numpy().astype(np.float32) == 256.5)


# one shape per tile at a depth the oracle cannot afford: 256 x 256 (eight waves, 128 half stages), the same tile with
# ragged edges and a K tail of 16, 128 x 128, 128 x 64, 64 x 64 with three buffers, and the register-staged kernel's range
@pytest.mark.parametrize("T,inp,out", [(4096, 4096, 4096), (8176, 4112, 8208), (4096, 4096, 2048), (2048, 6144, 3072),
                                       (512, 8192, 768), (16384, 768, 3072), (8192, 4080, 4096)])
def test_linear_dense_deep_k_closed_form(et, T, inp, out):
    """Small-integer operands with short periods: x[m, k] = (m + k) % 3 - 1, w[n, k] = (n + 2k) % 5 - 2, bias n % 4.
    Every product and partial sum is an integer below 2^24, so binary32 accumulation is exact in any order and
    the result depends on (m % 3, n % 5, n % 4) alone: the expected matrix is 15 sums, tiled, rounded once to
    binary16.  Bit-exact at full size: a stage multiplied from a buffer that was not ready, a tile mapped to the
    wrong place or a K tail handled wrongly all show."""
    k = np.arange(inp, dtype=np.int64)
    x = ((np.arange(T, dtype=np.int64)[:, None] + k[None, :]) % 3 - 1).astype(np.float16)
    w = ((np.arange(out, dtype=np.int64)[:, None] + 2 * k[None, :]) % 5 - 2).astype(np.float16)
    bias = (np.arange(out) % 4).astype(np.float16)
    sums = np.array([[int((((m + k) % 3 - 1) * ((n + 2 * k) % 5 - 2)).sum()) for n in range(5)] for m in range(3)], np.int32)
    want = sums[np.arange(T)[:, None] % 3, np.arange(out)[None, :] % 5] + (np.arange(out) % 4)[None, :]
    assert np.abs(want).max() < 2 ** 24
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.linear_dense(up(et, w), up(et, bias), up(et, x), d_y, T, inp, out)
    got = d_y.numpy()
    assert np.array_equal(got, want.astype(np.float32).astype(np.float16))


@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("M,N,K,batch", [(128, 64, 128, 12), (256, 768, 1536, 1), (48, 32, 16, 3),
                                         (128, 192, 1040, 3),  # long K in few tiles, 16 k-values in the last stage
                                         (32, 48, 400, 3)])    # batched small results
def test_gemm_batched(et, trans_b, M, N, K, batch):
    A = Hn.randn((batch, M, K), 4, 0.5)
    Bm = Hn.randn((batch, N, K) if trans_b else (batch, K, N), 5, 0.1)
    d_c = et.DeviceBuffer.empty((batch, M, N), np.float16)
    et.gemm(up(et, A), up(et, Bm), d_c, M, N, K, K, K if trans_b else N, N, trans_b, batch, M * K, Bm[0].size, M * N)
    Af, Bf = A.astype(np.float32), Bm.astype(np.float32)
    want = (Af @ (Bf.transpose(0, 2, 1) if trans_b else Bf)).astype(np.float16)
    assert Hn.max_abs(d_c.numpy(), want) <= 2e-2 * max(1.0, np.abs(want.astype(np.float32)).max() / 8)


def test_gemm_shared_operand_stride_zero(et):
    """stride 0 shares X between the problems of a batch (the Linear_VO call pattern)."""
    M, N, K, batch = 64, 48, 32, 5
    A, Bm = Hn.randn((M, K), 6, 0.5), Hn.randn((batch, K, N), 7, 0.1)
    d_c = et.DeviceBuffer.empty((batch, M, N), np.float16)
    et.gemm(up(et, A), up(et, Bm), d_c, M, N, K, K, N, N, False, batch, 0, K * N, M * N)
    want = (A.astype(np.float32)[None] @ Bm.astype(np.float32)).astype(np.float16)
    assert Hn.max_abs(d_c.numpy(), want) <= 4e-3


def test_gemm_rejects_bad_args(et):
    d = et.DeviceBuffer.empty((64, 64), np.float16)
    f = et.lib().et_gemm_f16
    assert f(d.ptr, d.ptr, d.ptr, 60, 64, 64, 64, 64, 64, 1, 1, 0, 0, 0, None) == et.ET_ERR_UNSUPPORTED
    assert f(d.ptr, d.ptr, d.ptr, 64, 64, 64, 32, 64, 64, 1, 1, 0, 0, 0, None) == et.ET_ERR_INVALID_ARG
    assert f(None, d.ptr, d.ptr, 64, 64, 64, 64, 64, 64, 1, 1, 0, 0, 0, None) == et.ET_ERR_INVALID_ARG
    assert f(d.ptr, d.ptr, d.ptr, 64, 64, 64, 64, 64, 64, 1, 0, 0, 0, 0, None) == et.ET_ERR_INVALID_ARG


@pytest.mark.parametrize("T,inp,out,sp,act", [(2048, 768, 768, 0.5, 0), (2048, 768, 3072, 0.5, 2),
                                              (2048, 3072, 768, 0.5, 0), (64, 64, 100 * 16, 0.9, 1),
                                              (8192, 128, 4096, 0.5, 2),  # the 256 x 256-tile kernel
                                              (2048, 720, 784, 0.45, 1),  # 432 surviving rows: a ragged tile edge
                                              (128, 768, 768, 0.9, 2),  # one sequence: the small-result kernel, scattered
                                              (2048, 768, 3072, 0.05, 2)])  # 2928 surviving rows: ragged 128 x 64 tiles, scattered
def test_linear_rowpruned(et, T, inp, out, sp, act):
    row_id = F.gen_row_ids(out, sp, seed=8)
    rows, b, x = Hn.randn((len(row_id), inp), 9, 0.02), Hn.randn((out,), 10, 0.1), Hn.randn((T, inp), 11)
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.check(et.lib().et_fill_f16(d_y.ptr, T * out, 0x7E00, None))  # every element must be written
    et.check(et.lib().et_linear_rowpruned_f16(up(et, rows).ptr, up(et, row_id).ptr, len(row_id), up(et, b).ptr,
                                              up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    want = L.linear_rowpruned(Hn.f32(x), Hn.f32(rows), row_id, out, Hn.f32(b), ACT[act], torch.float16).numpy()
    got = d_y.numpy()
    assert Hn.max_abs(got, want) <= 4e-3
    dead = np.setdiff1d(np.arange(out), row_id)
    bias_only = L.ACTS[ACT[act]](Hn.f32(b)).half().numpy()
    assert np.array_equal(got[:, dead], np.broadcast_to(bias_only[dead], (T, len(dead))))
    # compact output (the compact-V producer): column j = feature row_id[j], with its bias
    d_c = et.DeviceBuffer.empty((T, len(row_id)), np.float16)
    et.check(et.lib().et_linear_rowpruned_compact_f16(up(et, rows).ptr, up(et, row_id).ptr, len(row_id),
                                                      up(et, b).ptr, up(et, x).ptr, d_c.ptr, T, inp, None))
    want_c = L.linear(Hn.f32(x), Hn.f32(rows), Hn.f32(b[row_id]), None, torch.float16).numpy()
    assert Hn.max_abs(d_c.numpy(), want_c) <= 4e-3


@pytest.mark.parametrize("T,inp,out,sp,act", [(2048, 768, 768, 0.5, 0), (2048, 768, 3072, 0.5, 2),
                                              (2048, 3072, 768, 0.5, 0), (32, 160, 48, 0.3, 1), (128, 3072, 768, 0.9, 0)])
def test_linear_colpruned(et, T, inp, out, sp, act):
    col_id = F.gen_col_ids(inp, sp, seed=12)  # unsorted, as the reference generator leaves them
    cols, b, x = Hn.randn((out, len(col_id)), 13, 0.02), Hn.randn((out,), 14, 0.1), Hn.randn((T, inp), 15)
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.check(et.lib().et_linear_colpruned_f16(up(et, cols).ptr, up(et, col_id).ptr, len(col_id), up(et, b).ptr,
                                              up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    want = L.linear_colpruned(Hn.f32(x), Hn.f32(cols), col_id, Hn.f32(b), ACT[act], torch.float16).numpy()
    assert Hn.max_abs(d_y.numpy(), want) <= 4e-3
    # same result as the masked dense weight
    Wd = F.col_mat_to_dense(cols, col_id, inp)
    assert Hn.max_abs(want, L.linear(Hn.f32(x), Hn.f32(Wd), Hn.f32(b), ACT[act], torch.float16).numpy()) <= 2e-3
    # the workspace form: the gather is bit-exact, the Linear agrees with the oracle
    d_ws = et.DeviceBuffer.empty((T, len(col_id)), np.float16)
    d_y2 = et.DeviceBuffer.empty((T, out), np.float16)
    et.check(et.lib().et_linear_colpruned_ws_f16(up(et, cols).ptr, up(et, col_id).ptr, len(col_id), up(et, b).ptr,
                                                 up(et, x).ptr, d_y2.ptr, d_ws.ptr, T, inp, out, act, None))
    assert np.array_equal(d_ws.numpy(), x[:, col_id])
    assert Hn.max_abs(d_y2.numpy(), want) <= 4e-3


@pytest.mark.parametrize("T,inp,sp", [(2048, 768, 0.0), (2051, 768, 0.5), (1, 16, 0.0), (7, 3072, 0.9), (300, 8192, 0.5),
                                      (13, 1040, 0.3),
                                      # rows too long for the staged form: the lane-per-chunk kernel
                                      (5, 16400, 0.5), (64, 32768, 0.9)])
def test_gather_cols_is_exact(et, T, inp, sp):
    """Both column gathers (rows staged in LDS, and one chunk of eight a lane straight from memory)
    copy X[:, col_id] bit for bit, whatever the number of rows a workgroup ends on."""
    col_id = F.gen_col_ids(inp, sp, seed=T + inp)
    col_id = col_id[:len(col_id) // 8 * 8]
    x = Hn.randn((T, inp), 21)
    d_ws = et.DeviceBuffer.empty((T, len(col_id)), np.float16)
    et.check(et.lib().et_gather_cols_f16(d_ws.ptr, up(et, x).ptr, up(et, col_id).ptr, T, inp, len(col_id), None))
    assert np.array_equal(d_ws.numpy(), x[:, col_id])


@pytest.mark.parametrize("T,inp,out,sp,act", [(2048, 768, 768, 0.8, 0), (128, 768, 3072, 0.5, 2), (16, 32, 16, 0.0, 0),
                                              (80, 3072, 64, 0.9, 1)])
def test_linear_vec1x16(et, T, inp, out, sp, act):
    keep = np.repeat(torch.rand(out, inp // 16, generator=Hn.rng(16)).numpy() >= sp, 16, axis=1)
    W = (Hn.randn((out, inp), 17, 0.02).astype(np.float32) * keep).astype(np.float16)
    tile_idx, row_idx, data = F.dense_to_1x16(W)
    assert np.array_equal(F.mat1x16_to_dense(tile_idx, row_idx, data, out, inp), W)
    b, x = Hn.randn((out,), 18, 0.1), Hn.randn((T, inp), 19)
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    row_idx_d = row_idx if len(row_idx) else np.zeros(1, np.int32)
    et.check(et.lib().et_linear_vec1x16_f16(up(et, tile_idx).ptr, up(et, row_idx_d).ptr, up(et, data).ptr, up(et, b).ptr,
                                            up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    want = L.linear(Hn.f32(x), Hn.f32(W), Hn.f32(b), ACT[act], torch.float16).numpy()
    assert Hn.max_abs(d_y.numpy(), want) <= 4e-3
    # the dense image written on the device (what Linear<mat1x16> multiplies with) is exact
    d_w = et.DeviceBuffer.empty((out, inp), np.float16)
    et.check(et.lib().et_fill_f16(d_w.ptr, out * inp, 0x7E00, None))
    et.check(et.lib().et_vec1x16_to_dense_f16(up(et, tile_idx).ptr, up(et, row_idx_d).ptr, up(et, data).ptr, d_w.ptr,
                                              inp, out, None))
    assert np.array_equal(d_w.numpy(), W)  # as values: the masked W of this test holds -0.0 where the image has +0.0


def test_linear_vec1x16_unsorted_rows_in_a_cell(et):
    """Vectors of one (row-set, part) cell may come in any order (the seeded generator keeps the
    permuted order)."""
    T, inp, out = 32, 64, 32
    tile_idx, row_idx = F.gen_1x16_pattern(out, inp, 0.5, seed=3)
    data = Hn.randn((((len(row_idx) + 15) // 16) * 16, 16), 20, 0.1)
    W = F.mat1x16_to_dense(tile_idx, row_idx, data, out, inp)
    x = Hn.randn((T, inp), 21)
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.check(et.lib().et_linear_vec1x16_f16(up(et, tile_idx).ptr, up(et, row_idx).ptr, up(et, data).ptr, None,
                                            up(et, x).ptr, d_y.ptr, T, inp, out, 0, None))
    want = L.linear(Hn.f32(x), Hn.f32(W), None, None, torch.float16).numpy()
    assert Hn.max_abs(d_y.numpy(), want) <= 4e-3
    d_w = et.DeviceBuffer.empty((out, inp), np.float16)
    et.check(et.lib().et_vec1x16_to_dense_f16(up(et, tile_idx).ptr, up(et, row_idx).ptr, up(et, data).ptr, d_w.ptr,
                                              inp, out, None))
    assert np.array_equal(d_w.numpy(), W.astype(np.float16))


@pytest.mark.parametrize("T,inp,out,sp,act", [(1024, 768, 768, 0.9, 0), (100, 768, 3072, 0.95, 2), (7, 40, 12, 0.5, 1),
                                              (64, 40000, 16, 0.999, 0)])
def test_linear_csr(et, T, inp, out, sp, act):
    mask = torch.rand(out, inp, generator=Hn.rng(22)).numpy() >= sp
    W = (Hn.randn((out, inp), 23, 0.05).astype(np.float32) * mask).astype(np.float16)
    indptr, indices, data = F.dense_to_csr(W.astype(np.float32))
    b, x = Hn.randn((out,), 24, 0.1), Hn.randn((T, inp), 25)
    d_y = et.DeviceBuffer.empty((T, out), np.float16)
    et.check(et.lib().et_fill_f16(d_y.ptr, T * out, 0x7E00, None))
    et.check(et.lib().et_linear_csr_f16(up(et, indptr).ptr, up(et, indices).ptr, up(et, data.astype(np.float16)).ptr,
                                        up(et, b).ptr, up(et, x).ptr, d_y.ptr, T, inp, out, act, None))
    want = L.linear(Hn.f32(x), Hn.f32(W), Hn.f32(b), ACT[act], torch.float16).numpy()
    assert Hn.max_abs(d_y.numpy(), want) <= 4e-3


def test_linear_csr_reference_fixture(et):
    """The reference's dense_4_3.csr (all ones): y = sum of the 3 inputs + bias."""
    from pathlib import Path
    nrow, ncol, nnz, indptr, indices, data = F.read_csr(str(Path(__file__).parent / "golden" / "dense_4_3.csr"))
    x = Hn.randn((5, ncol), 26)
    b = np.array([0.5, -1, 2, 0], np.float16)
    d_y = et.DeviceBuffer.empty((5, nrow), np.float16)
    et.check(et.lib().et_linear_csr_f16(up(et, indptr).ptr, up(et, indices).ptr, up(et, data.astype(np.float16)).ptr,
                                        up(et, b).ptr, up(et, x).ptr, d_y.ptr, 5, ncol, nrow, 0, None))
    want = (x.astype(np.float32).sum(1, keepdims=True) + b.astype(np.float32)).astype(np.float16)
    assert Hn.max_abs(d_y.numpy(), want) <= 2e-3
