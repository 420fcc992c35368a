"""Shared helpers of the GPU parity tests, the smoke test and the bench:
seeded synthetic weights, upload/download, and oracle comparison."""
from __future__ import annotations

import hashlib
import math
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

from oracle import formats as F  # noqa: E402
from oracle import layers as L  # noqa: E402


# Device buffers created through up() stay alive until the test that made them ends
# (tests/conftest.py clears the list): a kernel launch is asynchronous, so a temporary
# whose raw pointer was passed to the C ABI must not be freed when the expression ends.
KEEP: list = []


def up(et, a):
    buf = et.DeviceBuffer.from_numpy(a)
    KEEP.append(buf)
    return buf


def rng(seed: int) -> torch.Generator:
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def randn(shape, seed, std=1.0, dtype=np.float16) -> np.ndarray:
    return (torch.randn(*shape, generator=rng(seed)) * std).numpy().astype(dtype)


def f32(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.asarray(a, dtype=np.float32))


def max_abs(a, b) -> float:
    return float(np.max(np.abs(np.asarray(a, np.float32) - np.asarray(b, np.float32)))) if np.size(a) else 0.0


class BsrWeight:
    """Seeded tile-sparse weight: pattern from the format oracle, values N(0, std)."""

    def __init__(self, out, inp, sparsity, seed, std=0.02, bias_std=0.0, dead_block_rows=(),
                 dead_block_cols=()):
        self.out, self.inp = out, inp
        self._pattern_args = (out, inp, sparsity, seed, tuple(dead_block_rows), tuple(dead_block_cols))
        # The index arrays live in anonymous mappings of their own, outside the malloc heap (see
        # isolated()).  The structure is frozen the moment it exists: numpy refuses any later
        # write through these arrays, and the digest taken here is compared again at every
        # hand-over to the library (check_tile_pattern), so a change made behind numpy's back
        # cannot go unseen.
        self.row_ptr, self.col_idx = self._generate_checked()
        bc = inp // 16
        assert len(self.col_idx) == 0 or (self.col_idx.min() >= 0 and self.col_idx.max() < bc), \
            "pattern generator produced a column tile outside the matrix"
        self.row_ptr.flags.writeable = False
        self.col_idx.flags.writeable = False
        self._pattern_digest = pattern_digest(self.row_ptr, self.col_idx)
        n = len(self.col_idx)
        self.tiles = randn((n, 256), seed + 1, std)
        self.bias = randn((out,), seed + 2, bias_std) if bias_std else np.zeros(out, np.float16)
        self.dense = F.bsr16_to_dense(self.row_ptr, self.col_idx, self.tiles, inp)  # fp16 values

    def _generate_checked(self):
        """The generator is deterministic, so two runs must agree; it works in small heap buffers, which is
        where this process has seen foreign writes (tests/heap_canary.py).  Two isolated copies that differ
        are written down and the structure is generated again until two consecutive runs agree."""
        prev = tuple(isolated(a) for a in self._pattern())
        for attempt in range(4):
            cur = tuple(isolated(a) for a in self._pattern())
            if all(np.array_equal(a, b) for a, b in zip(prev, cur)):
                return cur
            from tests import heap_canary
            for name, a, b in zip(("row_ptr", "col_idx"), prev, cur):
                bad = np.nonzero(a != b)[0]
                if len(bad):
                    heap_canary.note(
                        f"tile pattern {self._pattern_args}: two generations differ in {name} at {bad[:8].tolist()} "
                        f"(of {len(a)}): {a[bad[:8]].tolist()} against {b[bad[:8]].tolist()}, generation {attempt} and "
                        f"{attempt + 1}; generated again")
            prev = cur
        raise AssertionError(f"tile pattern {self._pattern_args}: no two consecutive generations agree")

    def _pattern(self):
        out, inp, sparsity, seed, dead_rows, dead_cols = self._pattern_args
        if dead_rows or dead_cols:
            return dead_aware_pattern(out, inp, sparsity, seed, dead_rows, dead_cols)
        return F.gen_tile_pattern(out, inp, sparsity, seed)

    def upload(self, et):
        check_tile_pattern(self, f"weight {self.out} x {self.inp}")
        self.d_row_ptr = et.DeviceBuffer.from_numpy(self.row_ptr)
        self.d_col_idx = et.DeviceBuffer.from_numpy(self.col_idx if len(self.col_idx) else np.zeros(1, np.int32))
        self.d_tiles = et.DeviceBuffer.from_numpy(self.tiles if len(self.tiles) else np.zeros((1, 256), np.float16))
        self.d_bias = et.DeviceBuffer.from_numpy(self.bias)
        return self

    def forward(self, et, dX, dY, T, act=0, stream=None):
        et.linear_bsr16(self.d_row_ptr, self.d_col_idx, self.d_tiles, self.d_bias, dX, dY, T,
                        self.inp, self.out, act, stream)


def dead_aware_pattern(out, inp, sparsity, seed, dead_block_rows, dead_block_cols):
    """Tile pattern with whole block-rows / block-columns removed (attention-aware
    pruning of V rows and the matching O columns); the surviving-tile count stays
    int(total*(1-sparsity)), chosen among the live positions in permuted order."""
    br, bc = out // 16, inp // 16
    total = br * bc
    ntile = F.tile_count(out, inp, sparsity)
    perm = F.permutation(total, seed)
    ys, xs = perm // bc, perm % bc
    live = ~np.isin(ys, list(dead_block_rows)) & ~np.isin(xs, list(dead_block_cols))
    kept = perm[live][:ntile]
    ys, xs = kept // bc, kept % bc
    row_ptr = np.zeros(br + 1, np.int32)
    cols = []
    for r in range(br):
        c = xs[ys == r]
        cols.append(c)
        row_ptr[r + 1] = row_ptr[r] + len(c)
    col_idx = np.concatenate(cols).astype(np.int32) if cols else np.zeros(0, np.int32)
    return row_ptr, col_idx


class LayerWeights:
    """One encoder layer: BSR Wqkv [3H,H], Wo [H,H], W1 [FF,H], W2 [H,FF] + LN params."""

    def __init__(self, H, nh, dimFF, sparsity, seed, attention_aware=0.0, bias_std=0.02):
        hd = H // nh
        dead_v, dead_o = (), ()
        if attention_aware > 0:
            # per head, the last `attention_aware` share of the V rows (16-row groups) is dead
            per_head_blocks = hd // 16
            ndead = int(per_head_blocks * attention_aware)
            dead_feat_blocks = [h * per_head_blocks + (per_head_blocks - 1 - i)
                                for h in range(nh) for i in range(ndead)]
            dead_v = tuple(2 * (H // 16) + b for b in dead_feat_blocks)  # V rows of Wqkv
            dead_o = tuple(dead_feat_blocks)                             # matching O input columns
        self.qkv = BsrWeight(3 * H, H, sparsity, seed * 100 + 1, bias_std=bias_std, dead_block_rows=dead_v)
        if dead_v:
            # a dead V feature has no weights and no bias
            for b in dead_v:
                self.qkv.bias[16 * b:16 * b + 16] = 0
        self.o = BsrWeight(H, H, sparsity, seed * 100 + 11, bias_std=bias_std, dead_block_cols=dead_o)
        self.l1 = BsrWeight(dimFF, H, sparsity, seed * 100 + 21, bias_std=bias_std)
        self.l2 = BsrWeight(H, dimFF, sparsity, seed * 100 + 31, bias_std=bias_std)
        self.g1 = (1.0 + randn((H,), seed * 100 + 41, 0.1, np.float32)).astype(np.float16)
        self.be1 = randn((H,), seed * 100 + 42, 0.1)
        self.g2 = (1.0 + randn((H,), seed * 100 + 43, 0.1, np.float32)).astype(np.float16)
        self.be2 = randn((H,), seed * 100 + 44, 0.1)
        self.H, self.nh, self.dimFF = H, nh, dimFF

    def oracle_params(self) -> L.LayerParams:
        return L.LayerParams(f32(self.qkv.dense), f32(self.qkv.bias), f32(self.o.dense), f32(self.o.bias),
                             f32(self.l1.dense), f32(self.l1.bias), f32(self.l2.dense), f32(self.l2.bias),
                             f32(self.g1), f32(self.be1), f32(self.g2), f32(self.be2))

    def upload(self, et):
        for w in (self.qkv, self.o, self.l1, self.l2):
            w.upload(et)
        self.d_g1, self.d_be1 = et.DeviceBuffer.from_numpy(self.g1), et.DeviceBuffer.from_numpy(self.be1)
        self.d_g2, self.d_be2 = et.DeviceBuffer.from_numpy(self.g2), et.DeviceBuffer.from_numpy(self.be2)
        return self


class LayerScratch:
    def __init__(self, et, T, H, dimFF):
        E = et.DeviceBuffer.empty
        self.qkv = E((T, 3 * H), np.float16)
        self.z = E((T, H), np.float16)
        self.attn = E((T, H), np.float16)
        self.ln1 = E((T, H), np.float16)
        self.ff = E((T, dimFF), np.float16)
        self.ff2 = E((T, H), np.float16)


def layer_forward_abi(et, w: LayerWeights, sc: LayerScratch, dX, dOut, B, S, d_lens=None, act=2,
                      eps=1e-5, flags=0, d_mask=None, stream=None):
    """One encoder layer through the kernel-level C ABI (the launch sequence the
    C++ Encoder class issues)."""
    H, nh = w.H, w.nh
    hd = H // nh
    T = B * S
    w.qkv.forward(et, dX, sc.qkv, T, 0, stream)
    q, k, v = sc.qkv.ptr, sc.qkv.offset(2 * H), sc.qkv.offset(4 * H)
    et.mha_fused(q, k, v, 3 * H, 3 * H, 3 * H, sc.z, H, d_mask, d_lens, B, S, nh, hd,
                 1.0 / math.sqrt(hd), flags, stream)
    w.o.forward(et, sc.z, sc.attn, T, 0, stream)
    et.skip_layernorm(sc.ln1, sc.attn, dX, w.d_g1, w.d_be1, T, H, eps, stream)
    w.l1.forward(et, sc.ln1, sc.ff, T, act, stream)
    w.l2.forward(et, sc.ff, sc.ff2, T, 0, stream)
    et.skip_layernorm(dOut, sc.ff2, sc.ln1, w.d_g2, w.d_be2, T, H, eps, stream)


def run_layer_case(et, H, nh, dimFF, S, B, sparsity, seed, lens=None, nlayers=1, attention_aware=0.0):
    """Runs nlayers encoder layers on the GPU and returns the max-abs error
    against the fp16-storage oracle."""
    T = B * S
    layers = [LayerWeights(H, nh, dimFF, sparsity, seed + i, attention_aware).upload(et) for i in range(nlayers)]
    x = randn((T, H), seed + 1000, 1.0)
    sc = LayerScratch(et, T, H, dimFF)
    bufs = [et.DeviceBuffer.from_numpy(x), et.DeviceBuffer.empty((T, H), np.float16)]
    d_lens = et.DeviceBuffer.from_numpy(np.asarray(lens, np.int32)) if lens is not None else None
    for i, w in enumerate(layers):
        layer_forward_abi(et, w, sc, bufs[i % 2], bufs[(i + 1) % 2], B, S, d_lens)
    got = bufs[nlayers % 2].numpy(np.float16, (T, H))
    cfg = L.LayerConfig(nh=nh, B=B, act="gelu", lens=None if lens is None else torch.as_tensor(lens),
                        store=torch.float16)
    want = L.encoder_stack(f32(x), [w.oracle_params() for w in layers], cfg).numpy()
    return max_abs(got, want)


def isolated(arr: np.ndarray) -> np.ndarray:
    """Copy of an index array in an anonymous private mapping of its own (whole pages, fresh from
    the kernel, never part of the malloc heap).  Twice a run of the GPU suite found a pattern
    changed after generation: two 8-byte words of a 920-byte numpy buffer, 736 bytes apart, each
    lower by exactly 6 — what decrements of a counter through dangling pointers into a freed and
    recycled heap block look like (both addresses were former 16-byte-aligned allocations with
    the word at offset 8).  This library has no such counter and its host code is clean under
    AddressSanitizer, so the writer is another component of the process; small numpy buffers come
    from the recycled heap, a private mapping cannot be the target of a pointer into it."""
    import mmap
    mm = mmap.mmap(-1, max(arr.nbytes, 1))
    out = np.frombuffer(mm, dtype=arr.dtype, count=arr.size)
    out[...] = arr
    return out


def pattern_digest(row_ptr, col_idx) -> str:
    return hashlib.sha1(row_ptr.tobytes() + col_idx.tobytes()).hexdigest()


def check_tile_pattern(bw, what):
    """A tile pattern must reach the library exactly as it was generated.  The arrays are
    read-only for numpy from the moment they exist, so a difference here means that memory
    was written behind numpy's back; the test stops and says where and what."""
    if pattern_digest(bw.row_ptr, bw.col_idx) == bw._pattern_digest:
        return
    bc = bw.inp // 16
    fresh_rp, fresh_ci = bw._pattern()
    bad = np.nonzero(bw.col_idx != fresh_ci)[0]
    bad_rp = np.nonzero(bw.row_ptr != fresh_rp)[0]
    lo = max(0, int(bad[0]) - 8) if len(bad) else 0
    raise AssertionError(
        f"{what}: the tile pattern changed after it was generated ({len(bad)} of {len(bw.col_idx)} column ids, "
        f"{len(bad_rp)} of {len(bw.row_ptr)} row pointers; {bc} column tiles): first at {bad[:8]}, values "
        f"{bw.col_idx[bad[:8]]} instead of {fresh_ci[bad[:8]]}, col_idx[{lo}:{lo + 40}] = {bw.col_idx[lo:lo + 40]}, "
        f"bytes {bw.col_idx[lo:lo + 40].tobytes().hex()}, array at {bw.col_idx.ctypes.data:#x} "
        f"(owns its data: {bw.col_idx.flags.owndata}, writeable: {bw.col_idx.flags.writeable})")


def build_model(et, layers, S, B, act=2, lens=None, use_graph=True, causal=False, eps=1e-5, mixed=False):
    """Encoder stack through et_model_* from a list of LayerWeights (exact fp16 bits)."""
    w0 = layers[0]
    m = et.Model(w0.H, w0.nh, w0.dimFF, S, len(layers), batch=B, act=act, eps=eps, causal=causal,
                 use_graph=use_graph, mixed=mixed)
    for i, w in enumerate(layers):
        for which, bw in ((et.W_QKV, w.qkv), (et.W_O, w.o), (et.W_FF1, w.l1), (et.W_FF2, w.l2)):
            check_tile_pattern(bw, f"layer {i} matrix {which}")
            m.set_bsr16(i, which, bw.row_ptr, bw.col_idx, bw.tiles, bw.bias)
        m.set_norm(i, 0, w.g1, w.be1)
        m.set_norm(i, 1, w.g2, w.be2)
    if lens is not None:
        m.set_lens(lens)
    m.finalize()
    return m


def oracle_stack(x, layers, B, lens=None, act="gelu", causal=False, eps=1e-5, store=torch.float16, resid="same",
                 boundary=None):
    """store=None: the fp32 mathematics; store=float16: fp16 at the engine's storage points;
    store=float16 with resid=float32: the engine's mixed-precision mode; with boundary=float16 as well:
    the class layer's forward(half*, half*), binary32 inside a layer and binary16 between layers."""
    cfg = L.LayerConfig(nh=layers[0].nh, B=B, act=act, eps=eps, causal=causal,
                        lens=None if lens is None else torch.as_tensor(np.asarray(lens)), store=store, resid=resid,
                        boundary=boundary)
    return L.encoder_stack(f32(x), [w.oracle_params() for w in layers], cfg).numpy()
