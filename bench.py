#!/usr/bin/env python3
"""Headline benchmark: 12-layer BERT-base encoder, fp16 storage / fp32 accumulation,
seq 128, batch 8, 80 % 16x16 tile sparsity with attention-aware V/O pruning.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one forward of the whole encoder stack over one batch of synthetic
token embeddings that already sit in HBM (one HIP-graph replay through the C ABI),
in the engine's mixed-precision mode: fp16 matrix-core operands, fp32 accumulation,
fp32 softmax, LayerNorm and residual stream.
Prints ONE JSON line: sequences/s (value), ms per step, per-layer latency, the
roofline of the dominant kernel — the launch with the largest share of the step's GPU time
in the committed rocprofv3 kernel trace: the tile-sparse FFN up-projection, 3072 x 768 at
80 %, which normalises the output projection's binary32 sum while it stages its token strip
and applies GELU in its epilogue (timed with HIP events on its own stream over a HIP graph
of such launches, each on another layer's weights and another set of buffers, so nothing
is warm in a cache) — and the CPU oracle timed on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

import __graft_entry__ as entry  # noqa: E402

# BERT-base encoder, the configuration the metric is quoted on
H, NH, FF, S, B, NLAYER = 768, 12, 3072, 128, 8, 12
SPARSITY = 0.8
ATTENTION_AWARE = 0.25

MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 matrix peak (vendor figure)
# HBM-side bytes per launch of the dominant kernel come from the committed PMC summary:
# rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (KiB per dispatch), each scaled by what the same
# counter reads for a streaming kernel of known size.  The summary ends in one machine-readable
# line, "bench.py reads: {json}", which is all this file takes from it; the kernel-trace summary
# ends in one such line too, with the profiler's average duration of the same kernel.
TRAFFIC_PROFILE = ROOT / "profiles" / "encoder_stack_bert_base_b8_s128_hbm_traffic.txt"
STATS_PROFILE = ROOT / "profiles" / "encoder_stack_bert_base_b8_s128_kernel_stats.txt"


def profile_line(path, kernel):
    """The dict of the 'bench.py reads:' line of a profile summary if it is about `kernel`, else (None, reason)."""
    try:
        for line in path.read_text().splitlines():
            if line.startswith("bench.py reads:"):
                d = json.loads(line.split(":", 1)[1])
                if d["kernel"] != kernel:
                    return None, f"{path.name} is about {d['kernel']}, not {kernel}"
                return d, d["kernel"]
    except (OSError, ValueError, KeyError) as e:
        return None, f"{path.name}: {e}"
    return None, f"{path.name}: no 'bench.py reads:' line"


def traffic_from_profile(kernel):
    """(bytes per launch, source note) of the dominant kernel, or (None, reason).  `kernel` is the
    instantiation the timed launch runs: counters of another one are not reported."""
    d, note = profile_line(TRAFFIC_PROFILE, kernel)
    if d is None:
        return None, note
    return (d["fetch_kib"] * d["fetch_factor"] + d["write_kib"] * d["write_factor"]) * 1024.0, note


class TileWeight:
    """One tile-sparse matrix of the workload, built with the library's own host routines
    (seeded permutation, surviving-tile count) and numpy: nothing here touches the CPU oracle."""

    def __init__(self, et, out, inp, seed, dead_block_rows=(), dead_block_cols=()):
        import ctypes as C
        lib = et.lib()
        br, bc = out // 16, inp // 16
        total = br * bc
        ntile = lib.et_fmt_kept_count(total, SPARSITY)  # int(total * (1.0 - (double)sparsity))
        perm = np.zeros(total, np.int64)
        et.check(lib.et_fmt_permutation(total, seed, perm.ctypes.data))
        ys, xs = perm // bc, perm % bc
        live = ~np.isin(ys, list(dead_block_rows)) & ~np.isin(xs, list(dead_block_cols))
        kept = perm[live][:ntile]  # surviving tiles among the live positions, in permuted order
        ys, xs = kept // bc, kept % bc
        order = np.argsort(ys, kind="stable")
        self.row_ptr = np.concatenate([[0], np.cumsum(np.bincount(ys, minlength=br))]).astype(np.int32)
        self.col_idx = xs[order].astype(np.int32)
        rng = np.random.default_rng(seed)
        self.tiles = (rng.standard_normal((len(kept), 256), dtype=np.float32) * 0.02).astype(np.float16)
        self.bias = (rng.standard_normal(out, dtype=np.float32) * 0.02).astype(np.float16)
        for r in dead_block_rows:  # a dead V feature has no weights and no bias
            self.bias[16 * r:16 * r + 16] = 0
        self.out, self.inp = out, inp

    def upload(self, et):
        D = et.DeviceBuffer.from_numpy
        self.d_row_ptr, self.d_col_idx = D(self.row_ptr), D(self.col_idx)
        self.d_tiles, self.d_bias = D(self.tiles), D(self.bias)
        return self


class LayerWeights:
    def __init__(self, et, seed):
        per_head = (H // NH) // 16
        ndead = int(per_head * ATTENTION_AWARE)
        dead = [h * per_head + (per_head - 1 - i) for h in range(NH) for i in range(ndead)]
        self.qkv = TileWeight(et, 3 * H, H, seed * 100 + 1, dead_block_rows=[2 * (H // 16) + b for b in dead])
        self.o = TileWeight(et, H, H, seed * 100 + 11, dead_block_cols=dead)
        self.l1 = TileWeight(et, FF, H, seed * 100 + 21)
        self.l2 = TileWeight(et, H, FF, seed * 100 + 31)
        rng = np.random.default_rng(seed * 100 + 41)
        g = lambda: (1.0 + 0.1 * rng.standard_normal(H, dtype=np.float32)).astype(np.float16)
        b = lambda: (0.1 * rng.standard_normal(H, dtype=np.float32)).astype(np.float16)
        self.g1, self.be1, self.g2, self.be2 = g(), b(), g(), b()


def build_layers(et):
    return [LayerWeights(et, 100 + i) for i in range(NLAYER)]


def build_model(et, layers, use_graph, mixed=1):
    # mixed precision: fp16 matrix-core operands, fp32 accumulation, fp32 residual stream / LayerNorm / softmax
    # (1: SkipLayerNorm folded into the neighbouring projections, 2: launched on its own)
    m = et.Model(H, NH, FF, S, NLAYER, batch=B, act=et.ACT_GELU, eps=1e-5, causal=False, use_graph=use_graph,
                 mixed=mixed)
    for i, w in enumerate(layers):
        for which, tw in ((et.W_QKV, w.qkv), (et.W_O, w.o), (et.W_FF1, w.l1), (et.W_FF2, w.l2)):
            m.set_bsr16(i, which, tw.row_ptr, tw.col_idx, tw.tiles, tw.bias)
        m.set_norm(i, 0, w.g1, w.be1)
        m.set_norm(i, 1, w.g2, w.be2)
    m.finalize()
    return m


def time_stack(et, model, d_out, d_in, steps, warmup):
    for _ in range(warmup):
        model.forward(d_out, d_in)
    model.sync()
    et.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        model.forward(d_out, d_in)
    model.sync()
    et.sync()
    return (time.perf_counter() - t0) / steps


def time_dominant_kernel(et, layers, T, folded, rounds_per_graph=6, replays=8):
    """(seconds per launch, kernel name as rocprofv3 prints it, description) of the stack's dominant
    kernel at the workload's shape: the FFN up-projection through the tile-sparse W1 (3072 x 768 at
    80 %) + GELU, T token rows, launched exactly as the stack launches it.

    `folded` (the default stack, four launches per layer): the launch normalises the output
    projection's binary32 sum V1 with that projection's row sums while it stages its token strip
    (et_norm_linear_bsr16_packed_f32in on a 12-wave pack, as the layer builds it); V1 and the sums are
    made here by the producer itself from random operands.  Otherwise (seven launches): the plain
    packed projection of a binary16 input.

    One HIP graph of rounds_per_graph x 12 launches, every launch on another layer's weights and
    its own buffers (nothing is warm in an L2 when a launch starts, as in the stack); all replays
    run between two HIP events on the launch stream, so no host launch latency is in the figure."""
    import ctypes as C
    lib = et.lib()
    stream = C.c_void_p()
    et.check(lib.et_stream_create(C.byref(stream)))
    rng = np.random.default_rng(0)
    n = len(layers)
    D = et.DeviceBuffer
    f16 = lambda *shape: D.from_numpy(rng.standard_normal(shape, dtype=np.float32).astype(np.float16))
    f32 = lambda *shape: D.from_numpy(rng.standard_normal(shape, dtype=np.float32))
    PRODUCER, CONSUMER = 2, 1  # ET_PACK_STATS_PRODUCER, ET_PACK_NORM_CONSUMER

    def pack(w, flags, nwave):
        h = C.c_void_p()
        et.check(lib.et_bsr16_pack_create(w.d_row_ptr.ptr, w.d_col_idx.ptr, w.d_tiles.ptr, T, w.inp, w.out, flags, nwave,
                                          C.byref(h)))
        return h

    for l in layers:
        for w in (l.o, l.l1):
            w.upload(et)
        l.d_g1, l.d_b1 = D.from_numpy(l.g1), D.from_numpy(l.be1)
    hs = [D.empty((T, FF), np.float16) for _ in layers]  # the up-projection's result
    if folded:
        po = [pack(l.o, PRODUCER, 12) for l in layers]
        p1 = [pack(l.l1, CONSUMER, 12) for l in layers]
        zs, x32 = [f16(T, H) for _ in layers], [f32(T, H) for _ in layers]
        v1 = [D.empty((T, H), np.float32) for _ in layers]
        st1 = [D.empty((16, T, 2), np.float32) for _ in layers]
        fin1 = [D.empty((T, 2), np.float32) for _ in layers]
        g1 = C.c_int(0)
        for i, l in enumerate(layers):
            et.check(lib.et_linear_bsr16_packed_resid_stats_f32(po[i], l.o.d_bias.ptr, zs[i].ptr, x32[i].ptr, None, None, None,
                                                                None, v1[i].ptr, st1[i].ptr, C.byref(g1), T, stream))
    else:
        po = []
        p1 = [pack(l.l1, 0, 0) for l in layers]
        y1s = [f16(T, H) for _ in layers]

    def up(i):
        l = layers[i]
        if folded:
            et.check(lib.et_norm_linear_bsr16_packed_f32in(p1[i], v1[i].ptr, st1[i].ptr, g1.value, l.d_g1.ptr, l.d_b1.ptr,
                                                           1e-5, fin1[i].ptr, l.l1.d_bias.ptr, hs[i].ptr, T, et.ACT_GELU,
                                                           stream))
        else:
            et.check(lib.et_linear_bsr16_packed_f16(p1[i], l.l1.d_bias.ptr, y1s[i].ptr, hs[i].ptr, None, T, et.ACT_GELU,
                                                    stream))

    info = [C.c_int() for _ in range(5)]
    et.check(lib.et_bsr16_pack_info(p1[0], *[C.byref(v) for v in info]))
    mt, ngroups, nwave, cap, _ = (v.value for v in info)
    su = 16 * mt * (H // 8) // (64 * nwave) if folded else 1  # strip vectors per thread of the normalising prologue
    name = (f"void et::bsr16_packed_kernel<{mt}, {cap}, {'true' if folded else 'false'}, false, {su}>(et::PackArgs)")
    what = (f"FFN up-projection 3072x768 @80% + GELU, T={T}, {nwave} waves x {cap} two-tile slots, "
            + ("normalising the output projection's binary32 sum while staging it" if folded else "binary16 input"))
    for i in range(n):  # eager once: one-time kernel setup
        up(i)
    et.check(lib.et_stream_sync(stream))
    et.check(lib.et_graph_begin_capture(stream))
    for _ in range(rounds_per_graph):
        for i in range(n):
            up(i)
    graph = C.c_void_p()
    et.check(lib.et_graph_end_capture(stream, C.byref(graph)))
    et.check(lib.et_graph_launch(graph, stream))  # warm
    et.check(lib.et_stream_sync(stream))
    with et.Timer(stream) as t:
        for _ in range(replays):
            et.check(lib.et_graph_launch(graph, stream))
    et.check(lib.et_graph_destroy(graph))
    et.check(lib.et_stream_sync(stream))
    for h in po + p1:
        et.check(lib.et_bsr16_pack_destroy(h))
    et.check(lib.et_stream_destroy(stream))
    return t.ms * 1e-3 / (rounds_per_graph * n * replays), name, what


def oracle_params(layers):
    import torch
    from oracle import formats as F
    from oracle import layers as L
    f32 = lambda a: torch.from_numpy(np.asarray(a, np.float32))
    dense = lambda w: f32(F.bsr16_to_dense(w.row_ptr, w.col_idx, w.tiles, w.inp))
    return [L.LayerParams(dense(w.qkv), f32(w.qkv.bias), dense(w.o), f32(w.o.bias), dense(w.l1), f32(w.l1.bias),
                          dense(w.l2), f32(w.l2.bias), f32(w.g1), f32(w.be1), f32(w.g2), f32(w.be2))
            for w in layers]


def oracle_forwards(layers, x):
    """(fp32 forward, forward with the engine's mixed-precision rounding points) of the workload."""
    import torch
    from oracle import layers as L
    params = oracle_params(layers)
    xt = torch.from_numpy(np.asarray(x, np.float32))
    with torch.no_grad():
        want32 = L.encoder_stack(xt, params, L.LayerConfig(nh=NH, B=B, act="gelu", store=None)).numpy()
        want_mixed = L.encoder_stack(xt, params, L.LayerConfig(nh=NH, B=B, act="gelu", store=torch.float16,
                                                               resid=torch.float32)).numpy()
    return want32, want_mixed


def cpu_baseline(layers, x, gpu_out, warmups=2, reps=5):
    """The CPU oracle (PyTorch-CPU fp32 forward, pruned weights as masked dense matrices) on
    the host cores: `warmups` untimed forwards, then the median of `reps` forwards of the full
    12-layer, batch-8 stack.  The only part of this file that uses oracle/: it also checks the GPU
    result of the same workload against the oracle."""
    import torch
    from oracle import layers as L

    # every host core this job may use: os.cpu_count(), capped by OMP_NUM_THREADS where the machine sets it
    # (a GPU box of the pool grants a one-GPU job 16 of the cores it reports and sets that variable)
    threads = os.cpu_count() or 1
    if os.environ.get("OMP_NUM_THREADS", "").isdigit():
        threads = max(1, min(threads, int(os.environ["OMP_NUM_THREADS"])))
    torch.set_num_threads(threads)
    params = oracle_params(layers)
    cfg = L.LayerConfig(nh=NH, B=B, act="gelu", store=None)
    xt = torch.from_numpy(np.asarray(x, np.float32))
    with torch.no_grad():
        for _ in range(warmups):
            L.encoder_stack(xt, params, cfg)
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            L.encoder_stack(xt, params, cfg)
            times.append(time.perf_counter() - t0)
    want32, want_mixed = oracle_forwards(layers, x)
    med = float(np.median(times))
    got = gpu_out.astype(np.float32)
    err32, errm = float(np.max(np.abs(got - want32))), float(np.max(np.abs(got - want_mixed)))
    refm = float(np.max(np.abs(want_mixed - want32)))
    return {"value": round(B / med, 3), "unit": "seq/s", "cores": torch.get_num_threads(), "host_cpu_count": os.cpu_count(),
            "kind": "port",
            "sample": f"{reps} forwards of the full workload (12 layers, batch 8, seq 128) after {warmups} warm-ups, "
                      f"median {med * 1e3:.1f} ms per forward, fp32 masked-dense PyTorch-CPU oracle",
            "us_per_layer": round(med * 1e6 / NLAYER, 1),
            # max-abs over the [1024 x 768] output of layer 12: the GPU (fp16 result) against the fp32 forward
            # timed above, against the same forward with the engine's rounding points (fp16 operands, fp32
            # residual stream), and those two against each other
            "gpu_max_abs_err_vs_fp32_forward": round(err32, 6),
            "gpu_max_abs_err_vs_mixed_precision_forward": round(errm, 6),
            "mixed_precision_forward_vs_fp32_forward": round(refm, 6)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--eager", action="store_true", help="launch kernel by kernel instead of replaying a graph")
    ap.add_argument("--separate-ln", action="store_true",
                    help="SkipLayerNorm as launches of its own (seven launches per layer) instead of folded into the "
                         "neighbouring projections (five)")
    ap.add_argument("--chain", action="store_true",
                    help="everything between two attention kernels in one launch (two launches per layer)")
    ap.add_argument("--five-launches", action="store_true",
                    help="the QKV projection as a launch of its own in every layer (five launches per layer) instead of "
                         "inside the attention kernel (four), which the engine picks for this batch by itself")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain streaming kernel of known size (ReLU over 64 MiB in, 64 MiB out) "
                         "three times, as the reference point for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this engine runs on ONE GPU (every sequence is independent; more GPUs would "
                 "replicate the weights and split the batch) — run with --gpus 1")

    et = entry.load_package()
    et.lib()  # fails loudly if the native library is missing

    layers = build_layers(et)
    model = build_model(et, layers, use_graph=not args.eager, mixed=2 if args.separate_ln else 3 if args.chain else 5 if args.five_launches else 1)
    x = np.random.default_rng(4).standard_normal((B * S, H), dtype=np.float32).astype(np.float16)
    d_in = et.DeviceBuffer.from_numpy(x)
    d_out = et.DeviceBuffer.empty((B * S, H), np.float16)

    sec = time_stack(et, model, d_out, d_in, args.steps, args.warmup)

    # dominant kernel (largest share of the step in the committed kernel trace): the FFN up-projection,
    # 3072x768 BSR at 80 %, T = 1024, + GELU; in the default stack it also normalises its input strip
    T = B * S
    folded = not args.separate_ln
    ntile = len(layers[0].l1.col_idx)  # the same count in every layer: int(9216 * (1 - 0.8))
    flops = 2.0 * 256 * ntile * T  # algorithmic: 2 * 16*16 * surviving tiles * token rows
    ksec, kname, kwhat = time_dominant_kernel(et, layers, T, folded)
    achieved = flops / ksec / 1e12
    traffic, traffic_note = traffic_from_profile(kname)
    prof, prof_note = profile_line(STATS_PROFILE, kname)
    roofline = {"bound": "mfma", "kernel": f"{kname}: {kwhat}",
                "achieved": round(achieved, 2), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 5), "us_per_launch": round(ksec * 1e6, 3),
                # the same kernel's average duration in the committed rocprofv3 kernel trace of this command: over
                # all its dispatches, and over those of the roofline loop timed here
                "us_per_launch_profile": None if prof is None else prof["avg_us"],
                "us_per_launch_profile_loop": None if prof is None else prof.get("loop_avg_us"),
                "profile_source": prof_note,
                "flop_per_launch": flops, "traffic": None if traffic is None else round(traffic),
                "traffic_source": traffic_note}
    # The same launch against the other roof: algorithmic bytes 2 T out (binary16 result) + 516 ntile +
    # 4 (out/16 + 1) + 2 out + the input strip: 2 T in as binary16, or folded 4 T in (the binary32 sum) +
    # 8 T groups (its row sums, 8 block-row groups) + 4 in (gamma, beta) + 8 T (row statistics written).
    # At about 100 flop per byte the shape sits below the ridge of the machine (312 flop/B), i.e. on the HBM roof.
    alg_bytes = 2.0 * T * FF + 516.0 * ntile + 4.0 * (FF // 16 + 1) + 2.0 * FF
    alg_bytes += (4.0 * T * H + 8.0 * T * 8 + 4.0 * H + 8.0 * T) if folded else 2.0 * T * H
    roofline["hbm_view"] = {"bound": "hbm", "achieved": round(alg_bytes / ksec / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                            "frac": round(alg_bytes / ksec / 8e12, 5), "bytes_per_launch": alg_bytes}

    out = {
        "metric": "BERT-base encoder seqs/sec + per-layer latency µs, seq128 fp16 80% tile-sparse",
        "value": round(B / sec, 2), "unit": "seq/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 5), "per_layer_us": round(sec * 1e6 / NLAYER, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "12-layer BERT-base encoder forward, H768 nh12 FFN3072, seq 128, batch 8, "
                               "80% 16x16 tile sparsity on Q/K/V/O/FFN, 25% of V rows / O columns pruned "
                               "in head-aligned groups, seeded N(0,0.02) weights, N(0,1) inputs",
                   "precision": "f16 matrix-core operands, f32 accumulation, f32 residual stream / LayerNorm / softmax "
                                "(wider than the all-f16 reference)",
                   "launch": "eager" if args.eager else "hip-graph",
                   "launches_per_layer": model.launches_per_layer()},
        "roofline": roofline,
    }
    if args.calibrate:
        n = 32 * 1024 * 1024  # fp16 elements: 64 MiB read, 64 MiB written per launch
        src = et.DeviceBuffer.from_numpy(np.ones(n, np.float16))
        dst = et.DeviceBuffer.empty((n,), np.float16)
        for _ in range(3):
            et.check(et.lib().et_relu_f16(dst.ptr, src.ptr, n, None))
        et.sync()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(layers, x, d_out.numpy())
    print(json.dumps(out))


if __name__ == "__main__":
    main()
