#!/usr/bin/env python3
"""Headline benchmark: 12-layer BERT-base encoder, fp16 storage / fp32 accumulation,
seq 128, batch 8, 80 % 16x16 tile sparsity with attention-aware V/O pruning.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one forward of the whole encoder stack over one batch of synthetic
token embeddings that already sit in HBM (one HIP-graph replay through the C ABI).
Prints ONE JSON line: sequences/s (value), ms per step, per-layer latency, the
roofline of the dominant kernel (SkipLayerNorm + tile-sparse FFN up-projection + GELU in
one launch, timed with HIP events on its own stream) and the CPU oracle timed on the host cores.
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
# HBM-side bytes per launch of the FFN up-projection kernel: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (KiB per dispatch), each scaled by what the same counter reads for a streaming
# kernel of known size (profiles/encoder_stack_bert_base_b8_s128_hbm_traffic.txt).
FFN_UP_TRAFFIC_BYTES = (5420.5 * 1.9989 + 7680.1 * 1.0) * 1024


def build_layers(Hn):
    return [Hn.LayerWeights(H, NH, FF, SPARSITY, seed=100 + i, attention_aware=ATTENTION_AWARE)
            for i in range(NLAYER)]


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


def time_ffn_kernel(et, w, T, launches_per_graph=64, replays=8):
    """Average duration of the layer's longest kernel at the workload's shape — y1 = SkipLayerNorm(
    attention output + layer input), then GELU(y1 W1^T + b1) through the tile-sparse W1, one
    launch: `launches_per_graph` launches recorded into one HIP graph, replayed between two HIP
    events on the same stream, so no host launch latency is in the figure."""
    import ctypes as C
    lib = et.lib()
    stream = C.c_void_p()
    et.check(lib.et_stream_create(C.byref(stream)))
    rng = np.random.default_rng(0)
    src = et.DeviceBuffer.from_numpy(rng.standard_normal((T, H)).astype(np.float16))
    skip = et.DeviceBuffer.from_numpy(rng.standard_normal((T, H)).astype(np.float16))
    gamma = et.DeviceBuffer.from_numpy(np.ones(H, np.float16))
    beta = et.DeviceBuffer.from_numpy(np.zeros(H, np.float16))
    y1 = et.DeviceBuffer.empty((T, H), np.float16)
    y = et.DeviceBuffer.empty((T, FF), np.float16)

    def launch():
        et.check(lib.et_skipln_linear_bsr16_f16(src.ptr, skip.ptr, gamma.ptr, beta.ptr, 1e-5, y1.ptr, w.d_row_ptr.ptr,
                                                w.d_col_idx.ptr, w.d_tiles.ptr, w.d_bias.ptr, y.ptr, T, H, FF,
                                                et.ACT_GELU, stream))

    launch()  # eager once (one-time kernel setup)
    et.check(lib.et_stream_sync(stream))
    et.check(lib.et_graph_begin_capture(stream))
    for _ in range(launches_per_graph):
        launch()
    graph = C.c_void_p()
    et.check(lib.et_graph_end_capture(stream, C.byref(graph)))
    et.check(lib.et_graph_launch(graph, stream))  # warm
    et.check(lib.et_stream_sync(stream))
    with et.Timer(stream) as t:
        for _ in range(replays):
            et.check(lib.et_graph_launch(graph, stream))
    et.check(lib.et_graph_destroy(graph))
    et.check(lib.et_stream_destroy(stream))
    return t.ms * 1e-3 / (launches_per_graph * replays)


def cpu_baseline(Hn, layers, x, reps=3):
    """The CPU oracle (PyTorch-CPU fp32 forward, pruned weights as masked dense matrices) on
    the host cores: one warm-up, then `reps` forwards of the full 12-layer, batch-8 stack."""
    import torch
    from oracle import layers as L

    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    params = [w.oracle_params() for w in layers]
    cfg = L.LayerConfig(nh=NH, B=B, act="gelu", store=None)
    xt = Hn.f32(x)
    with torch.no_grad():
        L.encoder_stack(xt, params, cfg)
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            L.encoder_stack(xt, params, cfg)
            times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(B / med, 3), "unit": "seq/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{reps} forwards of the full workload (12 layers, batch 8, seq 128) after 1 warm-up, "
                      f"median {med * 1e3:.1f} ms per forward, fp32 masked-dense PyTorch-CPU oracle",
            "us_per_layer": round(med * 1e6 / NLAYER, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--eager", action="store_true", help="launch kernel by kernel instead of replaying a graph")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain streaming kernel of known size (ReLU over 64 MiB in, 64 MiB out) "
                         "three times, as the reference point for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this engine runs on ONE GPU (every sequence is independent; more GPUs would "
                 "replicate the weights and split the batch) — run with --gpus 1")

    et = entry.load_package()
    et.lib()  # fails loudly if the native library is missing
    from tests import harness as Hn

    layers = build_layers(Hn)
    model = Hn.build_model(et, layers, S, B, act=et.ACT_GELU, use_graph=not args.eager)
    x = Hn.randn((B * S, H), 4)
    d_in = et.DeviceBuffer.from_numpy(x)
    d_out = et.DeviceBuffer.empty((B * S, H), np.float16)

    sec = time_stack(et, model, d_out, d_in, args.steps, args.warmup)

    # dominant kernel: SkipLayerNorm + FFN up-projection (3072x768 BSR at 80 %, T = 1024) + GELU
    T = B * S
    w1 = layers[0].l1.upload(et)
    ntile = len(layers[0].l1.col_idx)
    flops = 2.0 * 256 * ntile * T  # algorithmic: 2 * 16*16 * surviving tiles * token rows
    ksec = time_ffn_kernel(et, w1, T)
    achieved = flops / ksec / 1e12
    roofline = {"bound": "mfma", "kernel": "bsr16_linear_kernel<2,true,GELU,LN> SkipLayerNorm + 3072x768 @80% + GELU, T=1024",
                "achieved": round(achieved, 2), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 5), "us_per_launch": round(ksec * 1e6, 3),
                "flop_per_launch": flops, "traffic": round(FFN_UP_TRAFFIC_BYTES)}

    out = {
        "metric": "BERT-base encoder seqs/sec + per-layer latency µs, seq128 fp16 80% tile-sparse",
        "value": round(B / sec, 2), "unit": "seq/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 5), "per_layer_us": round(sec * 1e6 / NLAYER, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "12-layer BERT-base encoder forward, H768 nh12 FFN3072, seq 128, batch 8, "
                               "80% 16x16 tile sparsity on Q/K/V/O/FFN, 25% of V rows / O columns pruned "
                               "in head-aligned groups, seeded N(0,0.02) weights, N(0,1) inputs",
                   "launch": "eager" if args.eager else "hip-graph"},
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
        out["cpu_baseline"] = cpu_baseline(Hn, layers, x)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
