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


def cpu_baseline(gate, w, xs_host, logits_host, min_seconds):
    """candle's CPU path restated (the oracle: serial rows, columns threaded, AVX2 inner loops of
    candle's x86 build) on all host cores: the same batch, same weight bytes, same routing,
    repeated until `min_seconds` of wall time have passed."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import pyoracle as O

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    layer = O.Layer(H, F, E, TOPK, Q4K, gate, w["w1"], w["w3"], w["w2"])
    layer.forward(xs_host[:1], logits=logits_host[:1], simd=True, threads=cores)  # warm the pages
    reps, t0 = 0, time.perf_counter()
    while True:
        layer.forward(xs_host, logits=logits_host, simd=True, threads=cores)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds:
            break
    return {"value": xs_host.shape[0] * reps / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "%d forward(s) of the same %d-token batch through the same layer in %.1f s "
                      "(AVX2 vec_dot, %d threads over output columns)" % (reps, xs_host.shape[0], dt, cores)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--stage-iters", type=int, default=50)
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

        # per-stage durations: HIP events recorded by the library between its launches, same stream
        stage = {k: 0.0 for k in layer.STAGES}
        for i in range(args.stage_iters):
            for k, v in layer.forward_timed(xs[i % 4], ys[i % 4]).items():
                stage[k] += v / args.stage_iters
    stage_us = {k: round(v * 1e3, 2) for k, v in stage.items()}

    # Roofline of the dominant kernel, the up projection (w1, w3 + SiLU): it streams w1 and w3 of
    # every active expert exactly once per launch; algorithmic bytes = Q4_K bytes of those matrices
    # plus the quantised activations it reads and the quantised intermediate it writes.
    up_bytes = n_active * (2 * H * F * 144 // 256) + B * (H + H // 256 * 36) + B * TOPK * (F + F // 256 * 36)
    achieved = up_bytes / (stage["up"] * 1e-3) / 1e9
    step_bytes = n_active * EXPERT_BYTES + E * H * 4 + 2 * B * H * 4
    out = {
        "metric": "MoE layer tokens/s (Mixtral-8x7B shape, Q4_K, decode)", "value": tokens_per_s, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 2: hidden 4096, ffn 14336, 8 experts, top-2, Q4_K weights, decode batch %d" % B,
                   "active_experts": n_active, "wall_ms_per_step": wall * 1e3 / args.steps, "stage_us": stage_us,
                   "step_algorithmic_bytes": step_bytes,
                   "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "roofline": {"bound": "hbm", "kernel": "q4k_up (w1, w3, SiLU, Q8K re-quantisation)", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_launch": up_bytes, "launch_us": stage_us["up"]},
    }
    if not args.no_cpu_baseline:
        layer.forward(xs[0], out=ys[0])
        torch.cuda.synchronize()
        out["cpu_baseline"] = cpu_baseline(gate, w, xs[0].cpu().numpy(), layer.last_logits(B), args.cpu_seconds)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
