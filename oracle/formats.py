"""numpy restatement of the reference's sparse weight containers (test oracle).

Conventions: a Linear weight is the PyTorch ``[out, in]`` matrix (``nrow = out``,
``ncol = in``), as in the reference's generators (Linear/gen_linear.hpp:2-6).
All index arrays are int32; everything here is compared bit-exactly with the
C++ host implementation.

The reference draws random structure with ``std::random_shuffle`` over libstdc++
``rand()`` (e.g. mat_type/tile_mat/tile_mat.cu:16), which is not reproducible.
This build replaces the shuffle by a seeded permutation — ``permutation(n,
seed)`` = indices sorted by a SplitMix64 key — and keeps every other step of the
generators (counts, truncation, grouping, ordering) as the reference has them.
"""
from __future__ import annotations

import struct

import numpy as np

TILE = 16
_U64 = np.uint64


# --------------------------------------------------------------------------
# seeded permutation
# --------------------------------------------------------------------------

def splitmix64(seed: int, n: int) -> np.ndarray:
    """Key i = SplitMix64 output number i+1 of the stream started at ``seed``."""
    with np.errstate(over="ignore"):
        z = _U64(seed & 0xFFFFFFFFFFFFFFFF) + (np.arange(1, n + 1, dtype=_U64) * _U64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> _U64(30))) * _U64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> _U64(27))) * _U64(0x94D049BB133111EB)
        z = z ^ (z >> _U64(31))
    return z


def permutation(n: int, seed: int) -> np.ndarray:
    """The build's stand-in for std::random_shuffle(iota(n)): ids by ascending key."""
    return np.argsort(splitmix64(seed, n), kind="stable").astype(np.int64)


def _kept_fraction_count(total: int, sparsity: float) -> int:
    """``int(total * (1.0 - sparsity))`` with ``sparsity`` a C float promoted to
    double, as in mat_type/tile_mat/tile_mat.cu:12 (and the other generators)."""
    return int(total * (1.0 - float(np.float32(sparsity))))


# --------------------------------------------------------------------------
# tile_mat: 16x16 BSR   (mat_type/tile_mat/tile_mat.h:3-58)
# --------------------------------------------------------------------------

def tile_count(nrow: int, ncol: int, sparsity: float) -> int:
    """Surviving tiles of gen_sparse_mat (mat_type/tile_mat/tile_mat.cu:9-12)."""
    return _kept_fraction_count((nrow // TILE) * (ncol // TILE), sparsity)


def dense_to_bsr16(W: np.ndarray):
    """Exporter semantics (example/npy2pt.py:75-109): block-rows in order,
    column tiles ascending, a tile is kept iff any element is non-zero; tile
    data row-major [16 out][16 in] flattened to 256."""
    W = np.asarray(W)
    br, bc = W.shape[0] // TILE, W.shape[1] // TILE
    row_ptr = [0]
    column = []
    data = []
    for i in range(br):
        kept = 0
        for j in range(bc):
            blk = W[TILE * i:TILE * i + TILE, TILE * j:TILE * j + TILE]
            if not np.all(blk == 0):
                data.append(np.array(blk).reshape(-1))
                column.append(j)
                kept += 1
        row_ptr.append(row_ptr[-1] + kept)
    data_arr = np.array(data, dtype=W.dtype).reshape(len(column), TILE * TILE)
    return np.array(row_ptr, np.int32), np.array(column, np.int32), data_arr


def bsr16_to_dense(row_ptr, column, data, ncol: int) -> np.ndarray:
    """Masked dense [out, in] matrix of a BSR weight (tile order inside a
    block-row is free, as in the kernel's sum, Linear/SPMM_tile.cu:277-283)."""
    row_ptr = np.asarray(row_ptr)
    data = np.asarray(data).reshape(-1, TILE, TILE)
    br = len(row_ptr) - 1
    W = np.zeros((br * TILE, ncol), dtype=data.dtype)
    for r in range(br):
        for t in range(row_ptr[r], row_ptr[r + 1]):
            c = int(column[t])
            W[TILE * r:TILE * r + TILE, TILE * c:TILE * c + TILE] = data[t]
    return W


def gen_tile_pattern(nrow: int, ncol: int, sparsity: float, seed: int):
    """Structure of tile_mat::gen_sparse_mat (mat_type/tile_mat/tile_mat.cu:7-40):
    tile ids 0..total-1 map to (x = id % blk_col_num, y = id / blk_col_num)
    (lib/Coord.h:6-14), are permuted, truncated to ntile, and grouped by
    block-row keeping the permuted order (so columns are unsorted)."""
    br, bc = nrow // TILE, ncol // TILE
    total = br * bc
    ntile = _kept_fraction_count(total, sparsity)
    kept = permutation(total, seed)[:ntile]
    ys, xs = kept // bc, kept % bc
    row_ptr = np.zeros(br + 1, np.int32)
    row_offset = np.empty(ntile, np.int32)
    pos = 0
    for r in range(br):
        cols = xs[ys == r]
        row_offset[pos:pos + len(cols)] = cols
        pos += len(cols)
        row_ptr[r + 1] = pos
    return row_ptr, row_offset


def gen_dense_tile_pattern(nrow: int, ncol: int):
    """tile_mat::gen_dense_mat (mat_type/tile_mat/tile_mat.cu:42-64)."""
    br, bc = nrow // TILE, ncol // TILE
    row_ptr = (np.arange(br + 1) * bc).astype(np.int32)
    row_offset = np.tile(np.arange(bc, dtype=np.int32), br)
    return row_ptr, row_offset


# --------------------------------------------------------------------------
# row_mat / col_mat   (mat_type/row_mat/row_mat.cu, mat_type/col_mat/col_mat.cu)
# --------------------------------------------------------------------------

def gen_row_ids(nrow: int, sparsity: float, seed: int) -> np.ndarray:
    """row_mat::gen_sparse_mat (mat_type/row_mat/row_mat.cu:14-25): the kept
    output rows, count padded up to a multiple of 16, ids ascending."""
    nn = _kept_fraction_count(nrow, sparsity)
    nn = ((nn // 16) + (1 if nn % 16 else 0)) * 16
    nn = min(nn, nrow)
    return np.sort(permutation(nrow, seed)[:nn]).astype(np.int32)


def gen_col_ids(ncol: int, sparsity: float, seed: int) -> np.ndarray:
    """col_mat::gen_sparse_mat (mat_type/col_mat/col_mat.cu:22-32): the kept
    input columns, count rounded DOWN to a multiple of 16 (integer division
    inside the ceil), ids in permuted (unsorted) order."""
    nn = _kept_fraction_count(ncol, sparsity)
    nn = 16 * (nn // 16)
    return permutation(ncol, seed)[:nn].astype(np.int32)


def head_ptr(col_id, nnz_col: int, nhead: int, full_dim: int) -> np.ndarray:
    """col_mat::set_metadata (mat_type/col_mat/col_mat.cu:34-58): for ascending
    ``col_id``, head h owns positions [head_ptr[h], head_ptr[h+1]) — the ids in
    [h*hd, (h+1)*hd)."""
    hd = full_dim // nhead
    out = [0]
    for h in range(nhead):
        hi = (h + 1) * hd
        i = out[-1]
        while i < nnz_col and col_id[i] < hi:
            i += 1
        out.append(i)
    if out[-1] != nnz_col:
        raise ValueError(f"head_ptr ends at {out[-1]}, expected {nnz_col}")
    return np.array(out, np.int32)


def row_mat_to_dense(rows, row_id, nrow: int) -> np.ndarray:
    W = np.zeros((nrow, rows.shape[1]), rows.dtype)
    W[np.asarray(row_id)] = rows
    return W


def col_mat_to_dense(cols, col_id, ncol: int) -> np.ndarray:
    W = np.zeros((cols.shape[0], ncol), cols.dtype)
    W[:, np.asarray(col_id)] = cols
    return W


# --------------------------------------------------------------------------
# mat1x16: 1x16 vector sparsity   (mat_type/mat1x16/mat1x16.h:5-22)
#
# The reference leaves this format unfinished (generators and kernel are
# broken stubs); the layout below is the one its kernel reads
# (Linear/SPMM1x16.cu:52-74): for row-set r (16 output rows) and part p (16
# input columns), vectors idx in [tile_idx[r*(npart+1)+p], tile_idx[r*(npart+1)+p+1])
# are live; row_idx[idx] % 16 is the row inside the set and data[16*idx : 16*idx+16]
# the 16 weights.  Offsets are global, ascending over (r, p).
# --------------------------------------------------------------------------

def dense_to_1x16(W: np.ndarray):
    nrow, ncol = W.shape
    npart = ncol // TILE
    tile_idx, row_idx, data = [], [], []
    count = 0
    for r in range(nrow // TILE):
        for p in range(npart):
            tile_idx.append(count)
            for i in range(TILE):
                vec = W[r * TILE + i, p * TILE:(p + 1) * TILE]
                if np.any(vec != 0):
                    row_idx.append(r * TILE + i)
                    data.append(np.array(vec))
                    count += 1
        tile_idx.append(count)
    ntile = count
    pad = ((ntile + 15) // 16) * 16  # data padded to a multiple of 16 vectors (mat1x16.cu:7-13,51)
    d = np.zeros((pad, TILE), W.dtype)
    if ntile:
        d[:ntile] = np.array(data)
    return np.array(tile_idx, np.int32), np.array(row_idx, np.int32), d


def mat1x16_to_dense(tile_idx, row_idx, data, nrow: int, ncol: int) -> np.ndarray:
    npart = ncol // TILE
    W = np.zeros((nrow, ncol), data.dtype)
    for r in range(nrow // TILE):
        base = r * (npart + 1)
        for p in range(npart):
            for idx in range(tile_idx[base + p], tile_idx[base + p + 1]):
                W[r * TILE + row_idx[idx] % TILE, p * TILE:(p + 1) * TILE] = data[idx]
    return W


def gen_1x16_pattern(nrow: int, ncol: int, sparsity: float, seed: int):
    """Seeded structure in the spirit of mat1x16::gen_sparse_mat
    (mat_type/mat1x16/mat1x16.cu:38-75): vector ids over the (row, part) grid
    (x = id % npart, y = id / npart) permuted and truncated; inside one
    (row-set, part) cell the vectors keep the permuted order."""
    npart = ncol // TILE
    total = npart * nrow
    ntile = _kept_fraction_count(total, sparsity)
    kept = permutation(total, seed)[:ntile]
    ys, xs = kept // npart, kept % npart
    tile_idx, row_idx = [], []
    count = 0
    for r in range(nrow // TILE):
        in_set = (ys // TILE) == r
        for p in range(npart):
            tile_idx.append(count)
            rows = ys[in_set & (xs == p)]
            row_idx.extend(int(v) for v in rows)
            count += len(rows)
        tile_idx.append(count)
    return np.array(tile_idx, np.int32), np.array(row_idx, np.int32)


# --------------------------------------------------------------------------
# csr_mat   (mat_type/csr_mat/csr_mat.h:11-42)
# --------------------------------------------------------------------------

def dense_to_csr(W: np.ndarray):
    """Row-major scan, columns ascending, entry kept iff non-zero
    (mat_type/csr_mat/dense2csr.py:27-32 writes scipy's csr_matrix fields)."""
    indptr = [0]
    indices, data = [], []
    for r in range(W.shape[0]):
        nz = np.nonzero(W[r])[0]
        indices.extend(int(c) for c in nz)
        data.extend(W[r, nz].tolist())
        indptr.append(len(indices))
    return np.array(indptr, np.int32), np.array(indices, np.int32), np.array(data, np.float32)


def csr_to_dense(indptr, indices, data, ncol: int) -> np.ndarray:
    nrow = len(indptr) - 1
    W = np.zeros((nrow, ncol), np.float32)
    for r in range(nrow):
        for k in range(indptr[r], indptr[r + 1]):
            W[r, indices[k]] = data[k]
    return W


def gen_csr_pattern(nrow: int, ncol: int, sparsity: float, seed: int):
    """csr_mat::gen_sparse_mat (mat_type/csr_mat/csr_mat.cpp:25-67) with the
    column taken as id % ncol (the reference's ``i & ncol`` is a typo): ids
    permuted, truncated to nnz, grouped by row keeping the permuted order."""
    total = nrow * ncol
    nnz = _kept_fraction_count(total, sparsity)
    kept = permutation(total, seed)[:nnz]
    ys, xs = kept // ncol, kept % ncol
    indptr = np.zeros(nrow + 1, np.int32)
    indices = np.empty(nnz, np.int32)
    pos = 0
    for r in range(nrow):
        cols = xs[ys == r]
        indices[pos:pos + len(cols)] = cols
        pos += len(cols)
        indptr[r + 1] = pos
    return indptr, indices


# --------------------------------------------------------------------------
# file formats (little-endian, raw)
# --------------------------------------------------------------------------

def read_csr(path: str):
    """``u32 nrow,ncol,nnz; i32 indptr[nrow+1]; i32 indices[nnz]; f32 data[nnz]``
    (mat_type/csr_mat/csr_mat.h:19-35)."""
    raw = open(path, "rb").read()
    nrow, ncol, nnz = struct.unpack_from("<3I", raw, 0)
    off = 12
    indptr = np.frombuffer(raw, "<i4", nrow + 1, off); off += 4 * (nrow + 1)
    indices = np.frombuffer(raw, "<i4", nnz, off); off += 4 * nnz
    data = np.frombuffer(raw, "<f4", nnz, off)
    return nrow, ncol, nnz, indptr.copy(), indices.copy(), data.copy()


def write_csr(path: str, nrow, ncol, indptr, indices, data) -> None:
    with open(path, "wb") as f:
        f.write(struct.pack("<3I", nrow, ncol, len(indices)))
        f.write(np.asarray(indptr, "<i4").tobytes())
        f.write(np.asarray(indices, "<i4").tobytes())
        f.write(np.asarray(data, "<f4").tobytes())


def write_row_mat(path: str, nrow, ncol, row_id, rows) -> None:
    """``u32 nrow,ncol,len_id; i32 row_id[len_id]; f32 rows[len_id*ncol]``
    (mat_type/row_mat/gen_mat.py:17-29, read by row_mat.hpp:15-29)."""
    with open(path, "wb") as f:
        f.write(struct.pack("<3I", nrow, ncol, len(row_id)))
        f.write(np.asarray(row_id, "<i4").tobytes())
        f.write(np.asarray(rows, "<f4").tobytes())


def write_col_mat(path: str, nrow, ncol, col_id, cols) -> None:
    """``i32 nrow,ncol,len_id; i32 col_id[len_id]; f32 cols[nrow*len_id]``
    (mat_type/col_mat/col_mat.hpp:22-36)."""
    with open(path, "wb") as f:
        f.write(struct.pack("<3i", nrow, ncol, len(col_id)))
        f.write(np.asarray(col_id, "<i4").tobytes())
        f.write(np.asarray(cols, "<f4").tobytes())


def save_weight_npz(path: str, W: np.ndarray, B: np.ndarray) -> None:
    """One layer file of the exporter (example/npy2pt.py:112-119): a 2-D weight
    becomes row_ptr/column/data/B, a 1-D (LayerNorm) weight W/B; all float32."""
    if W.ndim == 2:
        row_ptr, column, data = dense_to_bsr16(W)
        np.savez(path, row_ptr=row_ptr, column=column, data=data.astype(np.float32),
                 B=B.astype(np.float32))
    else:
        np.savez(path, W=W.astype(np.float32), B=B.astype(np.float32))
