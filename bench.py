#!/usr/bin/env python3
"""Benchmark of the quantized sparse-MoE block on one MI355X.

Workload (BASELINE config 2): one Mixtral-8x7B-shape MoE layer, hidden 4096, expert FFN 14336,
8 experts, top-2, Q4_K weights (N(0, 0.02) quantised with candle's algorithm), f32 router gate,
decode batch of 32 tokens of N(0, 1) activations.  A "step" is one forward of the layer with the
activations already resident in HBM.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 32] [--no-cpu-baseline]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

H, F, E, TOPK = 4096, 14336, 8, 2
Q4K = 12
EXPERT_BYTES = 3 * H * F * 144 // 256          # 99,090,432 B of Q4_K blocks per expert
HBM_PEAK_GBS = 8000.0                          # MI355X HBM3E, published


def build_layer(torch, candle_amd, seed=0):
    """Weights drawn on the GPU, quantised there with the library's QTensor::quantize kernel
    (bit-identical to candle's CPU quantiser), kept as host bytes for the CPU baseline too."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    w = {"w1": [], "w3": [], "w2": []}
    for e in range(E):
        for name, shape in (("w1", (F, H)), ("w3", (F, H)), ("w2", (H, F))):
            x = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * 0.02
            w[name].append(candle_amd.quantize_weights(Q4K, x).cpu().numpy())
            del x
    g.manual_seed(seed + 1)
    gate = (torch.randn((E, H), generator=g, device="cuda", dtype=torch.float32) * 0.02).cpu().numpy()
    layer = candle_amd.SparseMoeBlock(H, F, E, TOPK, Q4K, gate, w["w1"], w["w3"], w["w2"])
    return layer, gate, w


def hip_events():
    """HIP events on an explicit stream via ctypes (torch's events only see torch's streams)."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipEventSynchronize.argtypes = [C.c_void_p]
    hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
    return hip


def cpu_baseline(gate, w, xs_host, logits_host, sample_experts):
    """candle's CPU path restated (oracle, AVX2 inner loops, all host cores) on a bounded sample:
    the same 32-token batch, but only the first `sample_experts` experts' token lists are run."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import pyoracle as O

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    probs = O.softmax_last_dim(logits_host)
    idx, wts, offsets, perm, perm_w = O.route(probs, TOPK)
    t0 = time.perf_counter()
    done_assign = 0
    for e in range(sample_experts):
        rows = perm[offsets[e]:offsets[e + 1]]
        if rows.size == 0:
            continue
        cur = np.ascontiguousarray(xs_host[rows])
        a = O.matmul(Q4K, cur, w["w1"][e], F, simd=True, threads=cores)
        b = O.matmul(Q4K, cur, w["w3"][e], F, simd=True, threads=cores)
        sil = a / (1.0 + np.exp(-a))
        O.matmul(Q4K, (sil * b).astype(np.float32), w["w2"][e], H, simd=True, threads=cores)
        done_assign += rows.size
    dt = time.perf_counter() - t0
    total_assign = xs_host.shape[0] * TOPK
    # time for the whole batch scales with the number of (token, expert) assignments
    est_full = dt * total_assign / max(done_assign, 1)
    return {"value": xs_host.shape[0] / est_full, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "%d of %d (token, expert) assignments of the same batch (experts 0..%d), %.1f s of CPU time, "
                      "scaled to the full batch" % (done_assign, total_assign, sample_experts - 1, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-experts", type=int, default=2)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU only (no collectives, no sharding); --gpus %d is not supported" % args.gpus)

    import numpy as np
    import torch
    import candle_amd

    candle_amd.load_library()  # fails loudly if the HIP extension is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    B = args.batch
    layer, gate, w = build_layer(torch, candle_amd)
    g = torch.Generator(device="cuda")
    g.manual_seed(2)
    # several distinct activation batches, rotated, so that no step repeats the previous one's input
    xs = [torch.randn((B, H), generator=g, device="cuda", dtype=torch.float32) for _ in range(4)]
    ys = [torch.empty_like(x) for x in xs]

    stream = torch.cuda.Stream()
    hip = hip_events()
    with torch.cuda.stream(stream):
        for i in range(args.warmup):
            layer.forward(xs[i % 4], out=ys[i % 4])
        stream.synchronize()
        n_active = int((np.diff(layer.last_routing(B)[2]) > 0).sum())
        ev = [C.c_void_p() for _ in range(2)]
        for e in ev:
            hip.hipEventCreate(C.byref(e))
        sh = C.c_void_p(stream.cuda_stream)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        hip.hipEventRecord(ev[0], sh)
        for i in range(args.steps):
            layer.forward(xs[i % 4], out=ys[i % 4])
        hip.hipEventRecord(ev[1], sh)
        hip.hipEventSynchronize(ev[1])
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms = C.c_float()
        hip.hipEventElapsedTime(C.byref(ms), ev[0], ev[1])
    ms_per_step = ms.value / args.steps
    tokens_per_s = B / (ms_per_step * 1e-3)

    # Roofline of the dominant kernels (the two expert products stream every active expert's
    # weights exactly once): algorithmic bytes per step / time of a step.
    algo_bytes = n_active * EXPERT_BYTES + E * H * 4 + 2 * B * H * 4
    achieved = algo_bytes / (ms_per_step * 1e-3) / 1e9
    out = {
        "metric": "MoE layer tokens/s (Mixtral-8x7B shape, Q4_K, decode)", "value": tokens_per_s, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8 x int4 -> i32, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 2: hidden 4096, ffn 14336, 8 experts, top-2, Q4_K weights, decode batch %d" % B,
                   "active_experts": n_active, "wall_ms_per_step": wall * 1e3 / args.steps},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": None, "algorithmic_bytes_per_step": algo_bytes,
                     "note": "whole step (router + up + down + combine) timed with HIP events on the launch stream"},
    }
    if not args.no_cpu_baseline:
        layer.forward(xs[0], out=ys[0])
        torch.cuda.synchronize()
        out["cpu_baseline"] = cpu_baseline(gate, w, xs[0].cpu().numpy(), layer.last_logits(B), args.cpu_sample_experts)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
