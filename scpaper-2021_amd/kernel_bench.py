#!/usr/bin/env python3
"""Per-kernel throughput against the roofline that bounds it, through the C ABI.

    python scpaper-2021_amd/kernel_bench.py [--set configs|scale|vo|mha|qkv|fuseo|plan|machine|all] [--json FILE]

`configs` are the shapes of the benchmark configurations (attention block at batch
1/4/16, the tile/row/column-pruned Linears at 2048 token rows, the BERT-large-shaped
layer); `scale` are shapes large enough that launch latency no longer matters, which
is where a kernel's fraction of the machine peak means something.  Every kernel is
recorded N times into one HIP graph and the graph is replayed between two HIP events
on its stream, so the figure is device time per launch.

Work counted is ALGORITHMIC: 2*256*ntile*T flops for a tile-sparse Linear,
2*T*in*out for a dense one, 4*S*S*hd*nh*B for the attention core, and the bytes a
normalisation or activation must move (inputs read once, output written once).
Peaks: 2500 TFLOP/s dense fp16 matrix rate, 8 TB/s HBM (vendor figures, MI355X).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))

import __graft_entry__ as entry  # noqa: E402

MFMA_PEAK_TFLOPS = 2500.0
HBM_PEAK_TBS = 8.0


class Bench:
    def __init__(self):
        self.et = entry.load_package()
        self.lib = self.et.lib()
        self.stream = C.c_void_p()
        self.et.check(self.lib.et_stream_create(C.byref(self.stream)))
        self.rng = np.random.default_rng(0)
        self.rows = []

    def rnd(self, shape, std=1.0):
        return (self.rng.standard_normal(shape, dtype=np.float32) * std).astype(np.float16)

    def dev(self, a):
        return self.et.DeviceBuffer.from_numpy(a)

    def empty(self, shape):
        return self.et.DeviceBuffer.empty(shape, np.float16)

    def time_us(self, fn, launches, replays=3):
        et, lib, s = self.et, self.lib, self.stream
        fn()
        et.check(lib.et_stream_sync(s))
        et.check(lib.et_graph_begin_capture(s))
        for _ in range(launches):
            fn()
        g = C.c_void_p()
        et.check(lib.et_graph_end_capture(s, C.byref(g)))
        et.check(lib.et_graph_launch(g, s))
        et.check(lib.et_stream_sync(s))
        with et.Timer(s) as t:
            for _ in range(replays):
                et.check(lib.et_graph_launch(g, s))
        et.check(lib.et_graph_destroy(g))
        return t.ms * 1e3 / (launches * replays)

    def record(self, kernel, shape, us, work, bound):
        if bound == "mfma":
            achieved, peak, unit = work / us / 1e6, MFMA_PEAK_TFLOPS, "TFLOP/s"
        else:
            achieved, peak, unit = work / us / 1e6, HBM_PEAK_TBS, "TB/s"
        row = {"kernel": kernel, "shape": shape, "us": round(us, 2), "bound": bound,
               "achieved": round(achieved, 2), "peak": peak, "unit": unit, "frac": round(achieved / peak, 4)}
        self.rows.append(row)
        print(f"{kernel:<22} {shape:<44} {us:10.1f} us  {achieved:8.2f} {unit:<8} {100 * achieved / peak:5.1f} % of {bound} peak",
              flush=True)

    # ---- kernels -------------------------------------------------------------------
    def layernorm(self, rows, H, launches):
        et = self.et
        a, b, o = self.dev(self.rnd((rows, H))), self.dev(self.rnd((rows, H))), self.empty((rows, H))
        g = self.dev(np.ones(H, np.float16))
        us = self.time_us(lambda: et.skip_layernorm(o, a, b, g, g, rows, H, 1e-5, self.stream), launches)
        self.record("skip_layernorm", f"{rows} x {H}", us, 3 * rows * H * 2 + 4 * H, "hbm")
        us = self.time_us(lambda: et.layernorm(o, a, g, g, rows, H, 1e-5, self.stream), launches)
        self.record("layernorm", f"{rows} x {H}", us, 2 * rows * H * 2 + 4 * H, "hbm")

    def gelu(self, n, launches):
        a, o = self.dev(self.rnd((n,))), self.empty((n,))
        us = self.time_us(lambda: self.et.check(self.lib.et_gelu_f16(o.ptr, a.ptr, n, self.stream)), launches)
        self.record("gelu", f"{n} values", us, 2 * n * 2, "hbm")

    def mha(self, B, S, nh, hd, launches, lens=None):
        et = self.et
        H = nh * hd
        qkv, z = self.dev(self.rnd((B * S, 3 * H))), self.empty((B * S, H))
        d_lens = self.dev(np.asarray(lens, np.int32)) if lens is not None else None
        us = self.time_us(lambda: et.mha_fused(qkv.ptr, qkv.offset(2 * H), qkv.offset(4 * H), 3 * H, 3 * H, 3 * H,
                                               z, H, None, d_lens, B, S, nh, hd, hd ** -0.5, 0, self.stream), launches)
        pairs = B * S * S if lens is None else int(sum(int(n) * int(n) for n in lens))
        tag = "" if lens is None else " padded"
        self.record("mha_fused", f"B{B} S{S} nh{nh} hd{hd}{tag}", us, 4 * pairs * hd * nh, "mfma")

    def dense(self, T, n_in, n_out, launches):
        et = self.et
        W, x, y = self.dev(self.rnd((n_out, n_in), 0.02)), self.dev(self.rnd((T, n_in))), self.empty((T, n_out))
        us = self.time_us(lambda: et.linear_dense(W, None, x, y, T, n_in, n_out, 0, self.stream), launches)
        self.record("linear_dense", f"T{T} in{n_in} out{n_out}", us, 2 * T * n_in * n_out, "mfma")

    def tile_pattern(self, n_out, n_in, sparsity, seed):
        """Seeded random tile structure from the library's own generator."""
        total = (n_out // 16) * (n_in // 16)
        row_ptr = np.zeros(n_out // 16 + 1, np.int32)
        col = np.zeros(max(total, 1), np.int32)
        ntile = C.c_int()
        self.et.check(self.lib.et_fmt_tile_pattern(n_out, n_in, sparsity, seed, row_ptr.ctypes.data, col.ctypes.data,
                                                   C.byref(ntile)))
        return row_ptr, col[:max(ntile.value, 1)].copy(), ntile.value

    def ids(self, fn, n, sparsity, seed):
        out = np.zeros(n + 16, np.int32)
        count = C.c_int()
        self.et.check(fn(n, sparsity, seed, out.ctypes.data, C.byref(count)))
        return out[:count.value].copy()

    def bsr(self, T, n_in, n_out, sparsity, launches, entry="class"):
        """Tile-sparse Linear.  entry = "class": through the entry point Linear<tile_mat> picks for this shape
        (include/et/Linear.h: the dense image above half of the tiles, the streaming plan for wide inputs at many
        rows, the row-loop pack from 2048 rows on for inputs up to 1536 wide where its launch fills the chip, a pack up
        to 1024 rows where block-rows average 8 tiles and the input is wide or the rows are at least 256, else the plain call); "plain" / "plan" / "pack" / "row loop" force one."""
        et, lib = self.et, self.lib
        row_ptr, col, ntile = self.tile_pattern(n_out, n_in, sparsity, 5)
        d_rp, d_col = self.dev(row_ptr), self.dev(col)
        tiles = self.dev(self.rnd((max(ntile, 1), 256), 0.02))
        bias = self.dev(np.zeros(n_out, np.float16))
        x, y = self.dev(self.rnd((T, n_in))), self.empty((T, n_out))
        label_class = entry == "class"
        if entry == "class":
            kept = ntile * 256.0 / (n_in * n_out)
            if kept > 0.5:
                entry = "dense image"
            elif n_in >= 128 and (n_in > 5112 or (n_in >= 3072 and T >= 4096)):
                entry = "plan"
            elif T >= 2048 and n_in % 128 == 0 and n_in <= 1536:
                entry = "row loop"  # falls back below when its launch would not fill the chip
            elif T <= 1024 and n_in % 128 == 0 and n_in <= 4096 and ntile >= 8 * (n_out // 16) and (n_in >= 2048 or T >= 256):
                entry = "pack"
            else:
                entry = "plain"
        handle, destroy = C.c_void_p(), None
        if entry == "plan":
            et.check(lib.et_bsr16_plan_create(d_rp.ptr, d_col.ptr, tiles.ptr, T, n_in, n_out, 0, 0, 0, C.byref(handle)))
            destroy = lib.et_bsr16_plan_destroy
            fn = lambda: et.check(lib.et_linear_bsr16_planned_f16(handle, bias.ptr, x.ptr, y.ptr, None, T, 0, self.stream))
        elif entry in ("pack", "row loop"):
            st = lib.et_bsr16_pack_create(d_rp.ptr, d_col.ptr, tiles.ptr, T, n_in, n_out, 4 if entry == "row loop" else 0, 0,
                                          C.byref(handle))
            thin = False
            if st == 0 and entry == "row loop":
                mt, groups = C.c_int(), C.c_int()
                et.check(lib.et_bsr16_pack_info(handle, C.byref(mt), C.byref(groups), None, None, None))
                thin = -(-T // (16 * mt.value)) * groups.value < 256
            if st == et.ET_ERR_UNSUPPORTED or (thin and label_class):
                if st == 0:
                    et.check(lib.et_bsr16_pack_destroy(handle))
                entry = "plain"
            else:
                et.check(st)
                destroy = lib.et_bsr16_pack_destroy
                fn = lambda: et.check(lib.et_linear_bsr16_packed_f16(handle, bias.ptr, x.ptr, y.ptr, None, T, 0, self.stream))
        elif entry == "dense image":
            w = self.empty((n_out, n_in))
            et.check(lib.et_bsr16_to_dense_f16(d_rp.ptr, d_col.ptr, tiles.ptr, w.ptr, n_in, n_out, self.stream))
            fn = lambda: et.check(lib.et_linear_dense_f16(w.ptr, bias.ptr, x.ptr, y.ptr, T, n_in, n_out, 0, self.stream))
        if entry == "plain":
            fn = lambda: et.linear_bsr16(d_rp, d_col, tiles, bias, x, y, T, n_in, n_out, 0, self.stream)
        us = self.time_us(fn, launches)
        et.check(lib.et_stream_sync(self.stream))
        if destroy:
            et.check(destroy(handle))
        self.record(f"linear_bsr16 ({entry})", f"T{T} in{n_in} out{n_out} sparsity {sparsity}", us, 2 * 256 * ntile * T, "mfma")

    def fuseo(self, B, S, sparsity, launches, nh=12, hd=64, nset=12):
        """Fused attention followed by the tile-sparse output projection: the one launch (et_mha_fuseo_f16, with the
        number of waves picked and forced) against the two launches it replaces (the projection through the plain
        call and, where one exists for the shape, through a pack); every launch of a graph on another of `nset`
        weight sets, as the layers of a stack."""
        et, lib = self.et, self.lib
        H, T = nh * hd, B * S
        sets, ntile = [], 0
        for i in range(nset):
            row_ptr, col, ntile = self.tile_pattern(H, H, sparsity, 70 + i)
            d_rp, d_col = self.dev(row_ptr), self.dev(col)
            tiles = self.dev(self.rnd((max(ntile, 1), 256), 0.02))
            pack = C.c_void_p()
            if lib.et_bsr16_pack_create(d_rp.ptr, d_col.ptr, tiles.ptr, T, H, H, 0, 0, C.byref(pack)) != 0:
                pack = None
            sets.append((d_rp, d_col, tiles, pack))
        bias = self.dev(np.zeros(H, np.float16))
        qkv, z, out = self.dev(self.rnd((T, 3 * H))), self.empty((T, H)), self.empty((T, H))
        scale, n = hd ** -0.5, {"i": 0}
        q, k, v = qkv.ptr, qkv.offset(2 * H), qkv.offset(4 * H)

        def one_launch(waves):
            def fn():
                s = sets[n["i"] % nset]
                n["i"] += 1
                et.check(lib.et_mha_fuseo_f16_geom(q, k, v, 3 * H, 3 * H, 3 * H, z.ptr, H, None, None, B, S, nh, hd, scale, 0,
                                                   s[0].ptr, s[1].ptr, s[2].ptr, bias.ptr, out.ptr, H, waves, self.stream))
            return fn

        def two_launches(packed):
            def fn():
                s = sets[n["i"] % nset]
                n["i"] += 1
                et.check(lib.et_mha_fused_f16(q, k, v, 3 * H, 3 * H, 3 * H, z.ptr, H, None, None, B, S, nh, hd, scale, 0,
                                              self.stream))
                if packed:
                    et.check(lib.et_linear_bsr16_packed_f16(s[3], bias.ptr, z.ptr, out.ptr, None, T, 0, self.stream))
                else:
                    et.check(lib.et_linear_bsr16_f16(s[0].ptr, s[1].ptr, s[2].ptr, bias.ptr, z.ptr, out.ptr, T, H, H, 0,
                                                     self.stream))
            return fn

        work = 2 * 256 * ntile * T + 4 * B * S * S * hd * nh
        shape = f"B{B} S{S} nh{nh} hd{hd} sparsity {sparsity}"
        self.record("mha + O (two launches, plain)", shape, self.time_us(two_launches(False), launches), work, "mfma")
        if all(s[3] is not None for s in sets):
            self.record("mha + O (two launches, pack)", shape, self.time_us(two_launches(True), launches), work, "mfma")
        self.record("mha + O (one launch)", shape, self.time_us(one_launch(0), launches), work, "mfma")
        for waves in (1, 2, 4):
            if (S // 16) % waves == 0:
                self.record(f"mha + O (one launch, {waves} waves)", shape, self.time_us(one_launch(waves), launches), work, "mfma")
        for s in sets:
            if s[3] is not None:
                et.check(lib.et_bsr16_pack_destroy(s[3]))

    def qkv_mha(self, B, S, sparsity, launches, nh=12, hd=64, nset=12):
        """The consumer QKV projection followed by the fused attention (two launches) against the attention kernel
        that projects Q, K and V itself (et_norm_qkv_mha_f32in), on the binary32 sum and row statistics a producer
        leaves; every launch of a graph on another of `nset` weight sets, as the layers of a stack."""
        et, lib = self.et, self.lib
        H, T = nh * hd, B * S
        sets, ntile = [], 0
        for i in range(nset):
            row_ptr, col, ntile = self.tile_pattern(3 * H, H, sparsity, 50 + i)
            d_rp, d_col = self.dev(row_ptr), self.dev(col)
            tiles = self.dev(self.rnd((max(ntile, 1), 256), 0.02))
            heads, consumer = C.c_void_p(), C.c_void_p()
            et.check(lib.et_qkv_heads_pack_create(d_rp.ptr, d_col.ptr, tiles.ptr, H, nh, C.byref(heads)))
            if lib.et_bsr16_pack_create(d_rp.ptr, d_col.ptr, tiles.ptr, T, H, 3 * H, 1, 0, C.byref(consumer)) != 0:
                consumer = None
            sets.append((d_rp, d_col, tiles, heads, consumer))
        bias = self.dev(np.zeros(3 * H, np.float16))
        v32 = self.rnd((T, H)).astype(np.float32)
        groups = 4
        stats = np.zeros((groups, T, 2), np.float32)
        for gi in range(groups):
            blk = v32[:, gi * H // groups:(gi + 1) * H // groups].astype(np.float64)
            stats[gi, :, 0], stats[gi, :, 1] = blk.sum(1), (blk * blk).sum(1)
        d_v, d_st = self.dev(v32), self.dev(stats)
        gamma, beta = self.dev(np.ones(H, np.float16)), self.dev(np.zeros(H, np.float16))
        fin = et.DeviceBuffer.empty((T, 2), np.float32)
        z, qkv = self.empty((T, H)), self.empty((T, 3 * H))
        scale, n = hd ** -0.5, {"i": 0}

        def one_launch():
            s = sets[n["i"] % nset]
            n["i"] += 1
            et.check(lib.et_norm_qkv_mha_f32in(s[3], d_v.ptr, d_st.ptr, groups, gamma.ptr, beta.ptr, 1e-5, fin.ptr, bias.ptr,
                                               z.ptr, H, None, None, B, S, scale, 0, self.stream))

        def two_launches():
            s = sets[n["i"] % nset]
            n["i"] += 1
            if s[4] is not None:
                et.check(lib.et_norm_linear_bsr16_packed_f32in(s[4], d_v.ptr, d_st.ptr, groups, gamma.ptr, beta.ptr, 1e-5,
                                                               fin.ptr, bias.ptr, qkv.ptr, T, 0, self.stream))
            else:
                et.check(lib.et_norm_linear_bsr16_f32in(d_v.ptr, d_st.ptr, groups, gamma.ptr, beta.ptr, 1e-5, fin.ptr, None, None,
                                                        s[0].ptr, s[1].ptr, s[2].ptr, bias.ptr, qkv.ptr, T, H, 3 * H, 0,
                                                        self.stream))
            et.check(lib.et_mha_fused_f16(qkv.ptr, qkv.offset(2 * H), qkv.offset(4 * H), 3 * H, 3 * H, 3 * H, z.ptr, H, None,
                                          None, B, S, nh, hd, scale, 0, self.stream))

        work = 2 * 256 * ntile * T + 4 * B * S * S * hd * nh
        shape = f"B{B} S{S} nh{nh} hd{hd} sparsity {sparsity}"
        self.record("norm + QKV + mha (two launches)", shape, self.time_us(two_launches, 4 * nset), work, "mfma")
        if lib.et_norm_qkv_mha_f32in_supported(B, S, H, nh, hd) == 1:
            self.record("norm_qkv_mha (one launch)", shape, self.time_us(one_launch, 4 * nset), work, "mfma")
        et.check(lib.et_stream_sync(self.stream))
        for s in sets:
            et.check(lib.et_bsr16_pack_destroy(s[3]))
            if s[4] is not None:
                et.check(lib.et_bsr16_pack_destroy(s[4]))

    def machine(self):
        """What a kernel boundary costs and how fast a compute unit takes bytes in (et_probe_*): the two figures
        that bound a launch of a few hundred kilobytes per compute unit."""
        et, lib = self.et, self.lib
        ncu = et.device_info()["num_cu"]
        us = self.time_us(lambda: et.check(lib.et_probe_empty(ncu, 256, self.stream)), 200)
        print(f"empty launch of {ncu} workgroups inside a graph: {us:.2f} us per launch (a kernel boundary)", flush=True)
        self.rows.append({"kernel": "probe_empty", "shape": f"{ncu} workgroups", "us": round(us, 2)})
        src_bytes = 1 << 30  # above the 256 MB Infinity Cache
        src = et.DeviceBuffer(src_bytes)
        sink = et.DeviceBuffer(4 * 4096)
        for threads, vec in ((256, 16), (512, 16), (768, 16), (768, 32), (1024, 16)):
            per_wg = threads * vec * 16
            for shared, what in ((1, "lines shared by the workgroups of an XCD (L2 hits after the first touch)"),
                                 (0, "lines of its own (first touch: Infinity Cache or HBM)")):
                # own lines: a different part of the gigabyte for every launch of the graph, so nothing is warm
                calls = {"n": 0}

                def fn():
                    off = 0 if shared else (calls["n"] % 8) * ncu * per_wg
                    calls["n"] += 1
                    et.check(lib.et_probe_read(src.ptr + off, src_bytes - off, ncu, threads, vec, shared, sink.ptr, self.stream))
                us = self.time_us(fn, 40)
                gbs = per_wg / us / 1e3
                print(f"read probe: {ncu} workgroups x {threads} threads x {vec} x 16 B = {per_wg // 1024} KB per compute unit, {what}: "
                      f"{us:.2f} us per launch, {gbs:.0f} GB/s per compute unit (launch included), {gbs * ncu / 1e3:.1f} TB/s over the chip",
                      flush=True)
                self.rows.append({"kernel": "probe_read", "shape": f"{per_wg // 1024} KB/CU {threads} thr shared={shared}",
                                  "us": round(us, 2), "gb_s_per_cu": round(gbs, 1)})

    def rowcol(self, T, n_in, n_out, sparsity, launches):
        et, lib = self.et, self.lib
        row_id = self.ids(lib.et_fmt_row_ids, n_out, sparsity, 7)
        rows = self.dev(self.rnd((len(row_id), n_in), 0.02))
        d_ids = self.dev(np.asarray(row_id, np.int32))
        bias = self.dev(np.zeros(n_out, np.float16))
        x, y = self.dev(self.rnd((T, n_in))), self.empty((T, n_out))
        us = self.time_us(lambda: et.check(lib.et_linear_rowpruned_f16(rows.ptr, d_ids.ptr, len(row_id), bias.ptr,
                                                                      x.ptr, y.ptr, T, n_in, n_out, 0, self.stream)),
                          launches)
        self.record("linear_rowpruned", f"T{T} in{n_in} out{n_out} sparsity {sparsity}", us,
                    2 * T * n_in * len(row_id), "mfma")
        col_id = self.ids(lib.et_fmt_col_ids, n_in, sparsity, 8)
        cols = self.dev(self.rnd((n_out, len(col_id)), 0.02))
        d_cid = self.dev(np.asarray(col_id, np.int32))
        ws = self.empty((T, len(col_id)))  # gather once, then a dense GEMM over the compact activations
        us = self.time_us(lambda: et.check(lib.et_linear_colpruned_ws_f16(cols.ptr, d_cid.ptr, len(col_id), bias.ptr,
                                                                         x.ptr, y.ptr, ws.ptr, T, n_in, n_out, 0,
                                                                         self.stream)), launches)
        self.record("linear_colpruned", f"T{T} in{n_in} out{n_out} sparsity {sparsity}", us,
                    2 * T * len(col_id) * n_out, "mfma")


    def vec1x16(self, T, n_in, n_out, sparsity, launches):
        et, lib = self.et, self.lib
        cells = (n_out // 16) * (n_in // 16 + 1)
        tile_idx = np.zeros(cells, np.int32)
        row_idx = np.zeros(n_out * (n_in // 16) + 16, np.int32)
        ntile = C.c_int()
        et.check(lib.et_fmt_1x16_pattern(n_out, n_in, sparsity, 9, tile_idx.ctypes.data, row_idx.ctypes.data,
                                         C.byref(ntile)))
        n = ntile.value
        data = self.dev(self.rnd((((n + 15) // 16) * 16 + 16, 16), 0.02))
        d_ti, d_ri = self.dev(tile_idx), self.dev(row_idx[:max(n, 1)].copy())
        bias = self.dev(np.zeros(n_out, np.float16))
        x, y = self.dev(self.rnd((T, n_in))), self.empty((T, n_out))
        us = self.time_us(lambda: et.check(lib.et_linear_vec1x16_f16(d_ti.ptr, d_ri.ptr, data.ptr, bias.ptr, x.ptr, y.ptr,
                                                                    T, n_in, n_out, 0, self.stream)), launches)
        self.record("linear_vec1x16", f"T{T} in{n_in} out{n_out} sparsity {sparsity}", us, 2 * 16 * n * T, "mfma")
        # what the Linear<mat1x16> class runs: the dense image, written once, and the dense GEMM on it
        w = self.empty((n_out, n_in))
        us = self.time_us(lambda: et.check(lib.et_vec1x16_to_dense_f16(d_ti.ptr, d_ri.ptr, data.ptr, w.ptr, n_in, n_out,
                                                                      self.stream)), launches)
        self.record("vec1x16_to_dense", f"in{n_in} out{n_out} sparsity {sparsity}", us, 2 * n_in * n_out + 32 * n, "hbm")
        us = self.time_us(lambda: et.check(lib.et_linear_dense_f16(w.ptr, bias.ptr, x.ptr, y.ptr, T, n_in, n_out, 0,
                                                                  self.stream)), launches)
        self.record("linear_vec1x16 image", f"T{T} in{n_in} out{n_out} sparsity {sparsity}", us, 2 * 16 * n * T, "mfma")

    def csr(self, T, n_in, n_out, sparsity, launches):
        et, lib = self.et, self.lib
        indptr = np.zeros(n_out + 1, np.int32)
        indices = np.zeros(n_out * n_in, np.int32)
        nnz = C.c_int()
        et.check(lib.et_fmt_csr_pattern(n_out, n_in, sparsity, 10, indptr.ctypes.data, indices.ctypes.data, C.byref(nnz)))
        n = nnz.value
        d_ip, d_ix = self.dev(indptr), self.dev(indices[:max(n, 1)].copy())
        data = self.dev(self.rnd((max(n, 1),), 0.02))
        bias = self.dev(np.zeros(n_out, np.float16))
        x, y = self.dev(self.rnd((T, n_in))), self.empty((T, n_out))
        us = self.time_us(lambda: et.check(lib.et_linear_csr_f16(d_ip.ptr, d_ix.ptr, data.ptr, bias.ptr, x.ptr, y.ptr, T,
                                                                n_in, n_out, 0, self.stream)), launches)
        self.record("linear_csr", f"T{T} in{n_in} out{n_out} sparsity {sparsity}", us, 2 * n * T, "mfma")

    def mha_compactv(self, B, S, nh, hd, live_per_head, launches):
        """Attention-aware pruning: `live_per_head` of the hd value columns of every head survive."""
        et, lib = self.et, self.lib
        H = nh * hd
        col_id = np.concatenate([h * hd + np.arange(live_per_head) for h in range(nh)]).astype(np.int32)
        head_ptr = (np.arange(nh + 1) * live_per_head).astype(np.int32)
        nnz = len(col_id)
        qk, vc, z = self.dev(self.rnd((B * S, 2 * H))), self.dev(self.rnd((B * S, nnz))), self.empty((B * S, H))
        d_cid, d_hp = self.dev(col_id), self.dev(head_ptr)
        us = self.time_us(lambda: et.check(lib.et_mha_compactv_f16(qk.ptr, qk.offset(2 * H), vc.ptr, 2 * H, 2 * H, nnz,
                                                                  d_cid.ptr, d_hp.ptr, nnz, z.ptr, H, None, None, B, S,
                                                                  nh, hd, hd, hd ** -0.5, 0, self.stream)), launches)
        self.record("mha_compactv", f"B{B} S{S} nh{nh} hd{hd} live {live_per_head}", us,
                    2 * B * S * S * nh * (hd + live_per_head), "mfma")

    def mha_vo(self, B, S, nh, hd, N, launches):
        """Pre-multiplied value/output projection (Linear_VO) and the attention over it."""
        et, lib = self.et, self.lib
        H = nh * hd
        W, x = self.dev(self.rnd((nh, H, N), 0.02)), self.dev(self.rnd((B * S, H)))
        vo = self.empty((B * nh * S, N))
        wt = self.empty((nh, N, H))  # k-contiguous per head, as the Linear_VO classes keep it
        et.check(lib.et_transpose_heads_f16(wt.ptr, W.ptr, nh, H, N, self.stream))
        us = self.time_us(lambda: et.check(lib.et_linear_vo_t_f16(wt.ptr, None, x.ptr, vo.ptr, B, S, H, N, nh, self.stream)),
                          launches)
        self.record("linear_vo", f"B{B} S{S} H{H} N{N} nh{nh}", us, 2 * B * S * H * N * nh, "mfma")
        qk, p, out = self.dev(self.rnd((B * S, 2 * H))), self.empty((B * S, nh * S)), self.empty((B * S, N))
        us = self.time_us(lambda: et.check(lib.et_mha_vo_f16(qk.ptr, qk.offset(2 * H), 2 * H, 2 * H, vo.ptr, p.ptr, out.ptr,
                                                            None, None, None, None, B, S, nh, hd, N, N, hd ** -0.5, 0,
                                                            self.stream)), launches)
        self.record("mha_vo", f"B{B} S{S} nh{nh} hd{hd} N{N}", us, 2 * B * S * S * nh * (hd + N), "mfma")
        us = self.time_us(lambda: et.check(lib.et_linear_vo_keys_f16(wt.ptr, x.ptr, vo.ptr, B, S, H, N, nh, self.stream)),
                          launches)
        self.record("linear_vo_keys", f"B{B} S{S} H{H} N{N} nh{nh}", us, 2 * B * S * H * N * nh, "mfma")
        us = self.time_us(lambda: et.check(lib.et_mha_vo_otf_f16(qk.ptr, qk.offset(2 * H), 2 * H, 2 * H, vo.ptr, None,
                                                                out.ptr, None, None, None, None, B, S, nh, hd, N, N,
                                                                hd ** -0.5, 0, self.stream)), launches)
        self.record("mha_vo_otf", f"B{B} S{S} nh{nh} hd{hd} N{N}", us, 2 * B * S * S * nh * (hd + N), "mfma")

    def mha_unfused(self, B, S, nh, hd, launches):
        """Scores through memory: batched GEMM, stand-alone softmax, batched GEMM (the comparison line)."""
        et, lib = self.et, self.lib
        H = nh * hd
        qkv, z, p = self.dev(self.rnd((B * S, 3 * H))), self.empty((B * S, H)), self.empty((B * nh * S, S))
        us = self.time_us(lambda: et.check(lib.et_mha_unfused_f16(qkv.ptr, qkv.offset(2 * H), qkv.offset(4 * H), 3 * H, 3 * H,
                                                                 3 * H, z.ptr, H, p.ptr, None, None, B, S, nh, hd,
                                                                 hd ** -0.5, 0, self.stream)), launches)
        self.record("mha_unfused", f"B{B} S{S} nh{nh} hd{hd}", us, 4 * B * S * S * hd * nh, "mfma")

    def f32_layer_kernels(self, B, S, H, nh, FF, launches):
        """The binary32 twins at the shapes of the dense fp32 layer (fp32 matrix peak 157.3 TFLOP/s)."""
        et, lib = self.et, self.lib
        T = B * S
        f = lambda *shape: et.DeviceBuffer.from_numpy(self.rng.standard_normal(shape, dtype=np.float32) * 0.05)
        e = lambda *shape: et.DeviceBuffer.empty(shape, np.float32)
        for n_in, n_out in ((H, 3 * H), (H, H), (H, FF), (FF, H)):
            W, x, y = f(n_out, n_in), f(T, n_in), e(T, n_out)
            us = self.time_us(lambda: et.check(lib.et_linear_dense_f32(W.ptr, None, x.ptr, y.ptr, T, n_in, n_out, 0,
                                                                      self.stream)), launches)
            self.record_f32("linear_dense_f32", f"T{T} in{n_in} out{n_out}", us, 2 * T * n_in * n_out)
        qkv, z = f(T, 3 * H), e(T, H)
        us = self.time_us(lambda: et.check(lib.et_mha_fused_f32(qkv.ptr, qkv.offset(4 * H), qkv.offset(8 * H), 3 * H, 3 * H,
                                                               3 * H, z.ptr, H, None, None, B, S, nh, H // nh,
                                                               (H // nh) ** -0.5, 0, self.stream)), launches)
        self.record_f32("mha_fused_f32", f"B{B} S{S} nh{nh} hd{H // nh}", us, 4 * B * S * S * H)

    def stack(self, name, H, nh, FF, S, B, nlayer, sparsity, lens, replays=20, mixed=0):
        """A whole encoder stack through the model handle (one HIP-graph replay per forward): every
        Linear tile-sparse at `sparsity` with its own seeded pattern, right padding `lens` or None."""
        et = self.et
        m = et.Model(H, nh, FF, S, nlayer, batch=B, act=et.ACT_GELU, eps=1e-5, causal=False, use_graph=True, mixed=mixed)
        flops = 0
        for i in range(nlayer):
            for which, (o, n_in) in ((et.W_QKV, (3 * H, H)), (et.W_O, (H, H)), (et.W_FF1, (FF, H)), (et.W_FF2, (H, FF))):
                row_ptr, col, ntile = self.tile_pattern(o, n_in, sparsity, 1000 * i + which + 1)
                m.set_bsr16(i, which, row_ptr, col, self.rnd((max(ntile, 1), 256), 0.02), self.rnd((o,), 0.02))
                flops += 2 * 256 * ntile * B * S
            for which in (0, 1):
                m.set_norm(i, which, (1.0 + self.rnd((H,), 0.1).astype(np.float32)).astype(np.float16), self.rnd((H,), 0.1))
        pairs = B * S * S if lens is None else int(sum(int(n) * int(n) for n in lens))
        flops += nlayer * 4 * pairs * H
        if lens is not None:
            m.set_lens(lens)
        m.finalize()
        x, y = self.dev(self.rnd((B * S, H))), self.empty((B * S, H))
        for _ in range(3):
            m.forward(y, x)
        m.sync()
        import time
        t0 = time.perf_counter()
        for _ in range(replays):
            m.forward(y, x)
        m.sync()
        us = (time.perf_counter() - t0) * 1e6 / replays
        mode = "binary32 residual stream" if mixed else "all activations binary16"
        self.record("encoder_stack", f"{name}, {mode}, {m.launches_per_layer()} launches per layer: {B / us * 1e6:.0f} seq/s, "
                                     f"{us / nlayer:.1f} us per layer", us, flops, "mfma")

    def record_f32(self, kernel, shape, us, flops):
        achieved, peak = flops / us / 1e6, 157.3
        self.rows.append({"kernel": kernel, "shape": shape, "us": round(us, 2), "bound": "mfma_f32",
                          "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s", "frac": round(achieved / peak, 4)})
        print(f"{kernel:<22} {shape:<44} {us:10.1f} us  {achieved:8.2f} TFLOP/s {100 * achieved / peak:5.1f} % of fp32 mfma peak",
              flush=True)


def run_configs(b: Bench):
    rng = np.random.default_rng(1)
    for B in (1, 4, 16):  # attention block, right padding with lengths in [64, 128]
        b.mha(B, 128, 12, 64, 50)
        b.mha(B, 128, 12, 64, 50, lens=rng.integers(64, 129, B))
    for n_in, n_out in ((768, 768), (768, 3072), (3072, 768)):  # pruned Linears at 2048 token rows
        for sp in (0.8, 0.9):
            b.bsr(2048, n_in, n_out, sp, 50)
        b.rowcol(2048, n_in, n_out, 0.5, 20)
        b.dense(2048, n_in, n_out, 20)
    b.layernorm(1024, 768, 50)   # the 12-layer workload's SkipLayerNorm
    b.layernorm(2048, 1024, 50)  # BERT-large-shaped layer
    b.mha(4, 512, 16, 64, 20)
    b.mha(4, 512, 16, 64, 20, lens=rng.integers(256, 513, 4))
    for n_in, n_out in ((1024, 1024), (1024, 3072), (1024, 4096), (4096, 1024)):
        b.bsr(2048, n_in, n_out, 0.9, 50)
    # the other weight formats and attention variants at the same configurations
    for n_in, n_out in ((768, 768), (768, 3072), (3072, 768)):
        b.vec1x16(2048, n_in, n_out, 0.8, 20)
        b.csr(2048, n_in, n_out, 0.8, 10)
    b.mha_compactv(8, 128, 12, 64, 48, 50)  # 25 % of the value columns of every head pruned
    b.mha_vo(1, 128, 12, 64, 768, 20)
    b.mha_vo(4, 128, 12, 64, 384, 20)       # half of the VO columns pruned
    b.mha_unfused(4, 128, 12, 64, 20)
    b.f32_layer_kernels(1, 128, 768, 12, 3072, 20)
    # whole stacks: 12-layer BERT-base at batch 8 (80 %), 24-layer BERT-large shape at batch 4, 512 tokens,
    # right padding with lengths in [256, 512] (90 %)
    b.stack("BERT-base 12 layers S128 B8 80%", 768, 12, 3072, 128, 8, 12, 0.8, None)
    b.stack("BERT-large 24 layers S512 B4 90% padded", 1024, 16, 4096, 512, 4, 24, 0.9, rng.integers(256, 513, 4))


def run_scale(b: Bench):
    b.layernorm(65536, 768, 10)
    b.layernorm(131072, 1024, 10)
    b.gelu(128 * 1024 * 1024, 10)
    b.mha(64, 512, 16, 64, 10)
    b.mha(16, 2048, 16, 64, 5)
    b.mha(16, 2048, 8, 128, 5)
    b.dense(8192, 4096, 4096, 5)
    b.dense(16384, 8192, 8192, 3)
    b.bsr(16384, 768, 3072, 0.8, 10)
    b.bsr(16384, 3072, 768, 0.8, 10)
    b.bsr(16384, 4096, 4096, 0.5, 3)
    b.rowcol(16384, 4096, 4096, 0.5, 3)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--set", choices=("configs", "scale", "vo", "mha", "qkv", "fuseo", "plan", "machine", "all"), default="all")
    ap.add_argument("--json", default=None, help="also write the rows as JSON to this file")
    args = ap.parse_args()
    b = Bench()
    print(json.dumps(b.et.device_info()))
    if args.set in ("configs", "all"):
        print("# shapes of the benchmark configurations")
        run_configs(b)
    if args.set == "mha":
        print("# fused attention from the benchmark shape to 2048 keys")
        rng = np.random.default_rng(1)
        for B in (1, 8, 16):
            b.mha(B, 128, 12, 64, 50)
        b.mha(8, 128, 12, 64, 50, lens=rng.integers(64, 129, 8))
        b.mha(4, 512, 16, 64, 20)
        b.mha(64, 512, 16, 64, 10)
        b.mha(16, 2048, 16, 64, 5)
        b.mha(16, 2048, 8, 128, 5)
        b.mha(16, 2048, 32, 32, 5)
    if args.set == "qkv":
        print("# the QKV projection inside the attention kernel against the two launches it replaces (768-wide, 12 heads of 64)")
        for B, S, sp in ((4, 128, 0.8), (8, 128, 0.8), (8, 128, 0.9), (12, 128, 0.8), (16, 128, 0.8), (16, 128, 0.9), (24, 128, 0.8),
                         (32, 128, 0.8), (16, 64, 0.8), (32, 64, 0.8), (64, 32, 0.8)):
            b.qkv_mha(B, S, sp, 48)
    if args.set == "fuseo":
        print("# attention + tile-sparse output projection: one launch against the two it replaces (768-wide, 12 heads of 64)")
        for B, S, sp in ((1, 128, 0.8), (1, 384, 0.8), (2, 128, 0.8), (4, 128, 0.8), (8, 128, 0.8), (8, 128, 0.9), (16, 128, 0.8),
                         (32, 128, 0.8), (64, 128, 0.8), (4, 512, 0.8)):
            b.fuseo(B, S, sp, 48)
    if args.set == "vo":
        print("# pre-computed-VO attention: probabilities through memory (mha_vo) and on chip (mha_vo_otf)")
        for B, N in ((1, 768), (4, 384), (8, 768), (16, 768)):
            b.mha_vo(B, 128, 12, 64, N, 20)
        b.mha_vo(4, 512, 16, 64, 1024, 10)
    if args.set == "plan":
        print("# tile-sparse Linear: the plain call, the streaming plan and (where it applies) a pack, at the same shapes")
        for T, n_in, n_out in ((1024, 3072, 768), (2048, 3072, 768), (4096, 3072, 768), (16384, 3072, 768), (16384, 768, 3072),
                               (2048, 6144, 768)):
            for entry in ("plain", "plan", "pack"):
                if entry == "pack" and (T > 4096 or n_in > 4096):
                    continue
                b.bsr(T, n_in, n_out, 0.8, 10 if T >= 16384 else 30, entry=entry)
        print("# ... and the row-loop pack (weights resident in registers, strips double-buffered) against the plain call and the pack")
        for T, n_in, n_out in ((1024, 768, 3072), (2048, 768, 3072), (4096, 768, 3072), (16384, 768, 3072), (2048, 768, 768),
                               (16384, 768, 768), (2048, 768, 2304), (16384, 768, 2304), (16384, 1024, 4096)):
            for entry in ("plain", "pack", "row loop"):
                if entry == "pack" and T > 4096:
                    continue
                b.bsr(T, n_in, n_out, 0.8, 10 if T >= 16384 else 30, entry=entry)
    if args.set == "machine":
        print("# machine probes")
        b.machine()
    if args.set in ("scale", "all"):
        print("# shapes where launch latency no longer matters")
        run_scale(b)
    if args.json:
        Path(args.json).write_text(json.dumps(b.rows, indent=1))


if __name__ == "__main__":
    main()
