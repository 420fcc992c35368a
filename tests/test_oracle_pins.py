"""Pins of the format oracle that do not come from the oracle itself: published SplitMix64
outputs, structures derived by hand from a printed permutation, and hand-written fixtures of the
1x16 layout and of the raw weight files (tests/golden/*.json).  The C++ host implementation is
held to the same values."""
import ctypes as C
import json
from pathlib import Path

import numpy as np
import pytest

from oracle import formats as F

GOLDEN = Path(__file__).resolve().parent / "golden"


def test_splitmix64_published_outputs():
    # the reference implementation's stream from seed 0 (Vigna, splitmix64.c) ...
    assert [int(v) for v in F.splitmix64(0, 3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    # ... and from seed 1234567 (the widely reproduced five-value test vector)
    assert [int(v) for v in F.splitmix64(1234567, 5)] == [6457827717110365317, 3203168211198807973,
                                                           9817491932198370423, 4593380528125082431,
                                                           16408922859458223821]


def test_permutation_from_published_keys(et):
    # ascending keys of seed 0: 0x06C4.. (id 2) < 0x6E78.. (id 1) < 0xE220.. (id 0)
    assert F.permutation(3, 0).tolist() == [2, 1, 0]
    # seed 1234567: keys 6457.., 3203.., 9817.., 4593.., 16408.. -> ids by ascending key
    assert F.permutation(5, 1234567).tolist() == [1, 3, 0, 2, 4]
    for n, seed, want in ((3, 0, [2, 1, 0]), (5, 1234567, [1, 3, 0, 2, 4])):
        out = np.zeros(n, np.int64)
        et.check(et.lib().et_fmt_permutation(n, seed, out.ctypes.data))
        assert out.tolist() == want


# permutation(12, 7) = [1, 10, 8, 5, 7, 0, 9, 4, 6, 3, 2, 11] (pinned here; everything below is derived
# from it by hand).
PERM12_SEED7 = [1, 10, 8, 5, 7, 0, 9, 4, 6, 3, 2, 11]


def test_generated_structures_derived_by_hand(et):
    assert F.permutation(12, 7).tolist() == PERM12_SEED7
    # csr_mat::gen_sparse_mat (mat_type/csr_mat/csr_mat.cpp:25-67), 3 x 4 at 50 %: nnz = 6, the first six ids
    # 1, 10, 8, 5, 7, 0 are (row, col) = (0,1) (2,2) (2,0) (1,1) (1,3) (0,0); rows keep the shuffled order
    indptr, indices = F.gen_csr_pattern(3, 4, 0.5, 7)
    assert indptr.tolist() == [0, 2, 4, 6] and indices.tolist() == [1, 0, 1, 3, 2, 0]
    # tile_mat::gen_sparse_mat (mat_type/tile_mat/tile_mat.cu:7-40), 48 x 64 = 3 x 4 tiles at 50 %: same ids, tile
    # (block-row, block-col) as above, grouped by block-row in shuffled order
    row_ptr, row_offset = F.gen_tile_pattern(48, 64, 0.5, 7)
    assert row_ptr.tolist() == [0, 2, 4, 6] and row_offset.tolist() == [1, 0, 1, 3, 2, 0]
    # row_mat (row_mat.cu:14-25): 12 rows at 50 % -> 6, padded to 16, capped at 12: every row, ascending
    assert F.gen_row_ids(12, 0.5, 7).tolist() == list(range(12))
    # col_mat (col_mat.cu:22-32): 12 columns at 50 % -> 6 -> rounded DOWN to a multiple of 16 = 0
    assert F.gen_col_ids(12, 0.5, 7).tolist() == []
    # the C++ generators give the same structures
    lib = et.lib()
    ip, ix, cnt = np.zeros(4, np.int32), np.zeros(6, np.int32), C.c_int()
    et.check(lib.et_fmt_csr_pattern(3, 4, 0.5, 7, ip.ctypes.data, ix.ctypes.data, C.byref(cnt)))
    assert cnt.value == 6 and ip.tolist() == [0, 2, 4, 6] and ix.tolist() == [1, 0, 1, 3, 2, 0]
    rp, ro = np.zeros(4, np.int32), np.zeros(6, np.int32)
    et.check(lib.et_fmt_tile_pattern(48, 64, 0.5, 7, rp.ctypes.data, ro.ctypes.data, C.byref(cnt)))
    assert cnt.value == 6 and rp.tolist() == [0, 2, 4, 6] and ro.tolist() == [1, 0, 1, 3, 2, 0]


def test_1x16_pattern_derived_by_hand(et):
    # permutation(64, 11) starts 41, 39, 6, 56, 10, 4, 20, 36.  32 x 32 weight = 32 rows x 2 parts = 64 vector
    # slots, id -> (row = id // 2, part = id % 2); 87.5 % sparsity keeps 8: (20,1) (19,1) (3,0) (28,0) (5,0) (2,0)
    # (10,0) (18,0).  Row set 0: part 0 holds rows 3, 5, 2, 10 (shuffled order), part 1 nothing; row set 1:
    # part 0 rows 28, 18, part 1 rows 20, 19.
    assert F.permutation(64, 11)[:8].tolist() == [41, 39, 6, 56, 10, 4, 20, 36]
    tile_idx, row_idx = F.gen_1x16_pattern(32, 32, 0.875, 11)
    assert tile_idx.tolist() == [0, 4, 4, 4, 6, 8]
    assert row_idx.tolist() == [3, 5, 2, 10, 28, 18, 20, 19]
    ti, ri, cnt = np.zeros(6, np.int32), np.zeros(8, np.int32), C.c_int()
    et.check(et.lib().et_fmt_1x16_pattern(32, 32, 0.875, 11, ti.ctypes.data, ri.ctypes.data, C.byref(cnt)))
    assert cnt.value == 8 and ti.tolist() == [0, 4, 4, 4, 6, 8] and ri.tolist() == [3, 5, 2, 10, 28, 18, 20, 19]


def golden_1x16():
    g = json.loads((GOLDEN / "vec1x16_small.json").read_text())
    W = np.zeros((g["nrow"], g["ncol"]), np.float32)
    for row, part, vals in g["vectors"]:
        W[row, 16 * part:16 * part + 16] = vals
    data = np.zeros((g["data_vectors"], 16), np.float32)
    data[:len(g["data_first_vectors"])] = g["data_first_vectors"]
    return g, W, data


def test_1x16_layout_against_hand_written_fixture(et):
    g, W, data = golden_1x16()
    tile_idx, row_idx, d = F.dense_to_1x16(W)
    assert tile_idx.tolist() == g["tile_idx"] and row_idx.tolist() == g["row_idx"]
    assert d.shape == data.shape and np.array_equal(d, data)
    # the fixture read the way the reference kernel reads it gives W back
    back = F.mat1x16_to_dense(np.array(g["tile_idx"]), np.array(g["row_idx"]), data, g["nrow"], g["ncol"])
    assert np.array_equal(back, W)
    # a wrong stride of tile_idx (npart instead of npart + 1 per row set) would misplace row set 1
    assert g["tile_idx"][3] == g["tile_idx"][2]  # row set 1 starts where row set 0 ended, one slot later
    # the C++ converter
    ti, ri = np.zeros(6, np.int32), np.zeros(5, np.int32)
    dv, cnt = np.zeros((16, 16), np.float32), C.c_int()
    et.check(et.lib().et_fmt_dense_to_1x16(W.ctypes.data, 32, 32, ti.ctypes.data, ri.ctypes.data, dv.ctypes.data,
                                           C.byref(cnt)))
    assert cnt.value == 5 and ti.tolist() == g["tile_idx"] and ri.tolist() == g["row_idx"] and np.array_equal(dv, data)


def files_fixture():
    g = json.loads((GOLDEN / "pruned_files.json").read_text())
    return g, {k: bytes.fromhex(g[k]["hex"].replace(" ", "")) for k in ("row", "col", "csr")}


def test_raw_weight_files_against_hand_written_bytes(tmp_path, et):
    g, raw = files_fixture()
    r, c, s = g["row"], g["col"], g["csr"]
    F.write_row_mat(str(tmp_path / "a.row"), r["nrow"], r["ncol"], r["row_id"], np.array(r["rows"], np.float32))
    assert (tmp_path / "a.row").read_bytes() == raw["row"]
    F.write_col_mat(str(tmp_path / "a.col"), c["nrow"], c["ncol"], c["col_id"], np.array(c["cols"], np.float32))
    assert (tmp_path / "a.col").read_bytes() == raw["col"]
    F.write_csr(str(tmp_path / "a.csr"), s["nrow"], s["ncol"], s["indptr"], s["indices"], s["data"])
    assert (tmp_path / "a.csr").read_bytes() == raw["csr"]
    # readers: the oracle's and the C++ host routine's, on the hand-written bytes
    (tmp_path / "b.csr").write_bytes(raw["csr"])
    nrow, ncol, nnz, indptr, indices, data = F.read_csr(str(tmp_path / "b.csr"))
    assert (nrow, ncol, nnz) == (2, 3, 3) and indptr.tolist() == s["indptr"] and indices.tolist() == s["indices"]
    assert data.tolist() == s["data"]
    lib = et.lib()
    nr, nc, nz = C.c_int(), C.c_int(), C.c_int()
    ip, ix, dv = np.zeros(3, np.int32), np.zeros(3, np.int32), np.zeros(3, np.float32)
    et.check(lib.et_fmt_csr_read(str(tmp_path / "b.csr").encode(), C.byref(nr), C.byref(nc), C.byref(nz),
                                 ip.ctypes.data, ix.ctypes.data, dv.ctypes.data))
    assert (nr.value, nc.value, nz.value) == (2, 3, 3)
    assert ip.tolist() == s["indptr"] and ix.tolist() == s["indices"] and dv.tolist() == s["data"]
    # a header that does not describe the file is refused, not trusted
    (tmp_path / "c.csr").write_bytes(raw["csr"][:8] + (1000).to_bytes(4, "little") + raw["csr"][12:])
    assert lib.et_fmt_csr_read(str(tmp_path / "c.csr").encode(), C.byref(nr), C.byref(nc), C.byref(nz), None, None,
                               None) == et.ET_ERR_IO
    # dense images of the two pruned containers
    assert F.row_mat_to_dense(np.array(r["rows"], np.float32), r["row_id"], 4).tolist() == [[0, 0], [1, 2], [0, 0], [3, -0.5]]
    assert F.col_mat_to_dense(np.array(c["cols"], np.float32), c["col_id"], 4).tolist() == [[2, 0, 1, 0], [-0.5, 0, 3, 0]]
