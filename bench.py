#!/usr/bin/env python3
"""Benchmark of the quantized sparse-MoE block on one MI355X.

Workload (BASELINE config 2): one Mixtral-8x7B-shape MoE layer, hidden 4096, expert FFN 14336,
8 experts, top-2, Q4_K weights (N(0, 0.02) quantised with candle's algorithm), f32 router gate,
decode batch of 32 tokens of N(0, 1) activations.  A "step" is one forward of the layer with the
activations already resident in HBM.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 32] [--no-cpu-baseline]

`--workload prefill` measures BASELINE config 3 instead (same layer, 4096 tokens, router bias that makes
the expert load follow Zipf(1)); its roofline object is the int8-MFMA one of the tiled up kernel.
`--weights q4_0|q4_1|q5_0|q5_1|q8_0|q2_k|q3_k|q5_k|q6_k` runs the decode workload on the same layer shape with
another GGML format (random block payloads with small finite scales: timing does not depend on the values).
`--workload config4` measures BASELINE config 4 (hidden 2048, 60 experts of FFN 1408, top-4, one always-on
shared expert of FFN 5632 behind a sigmoid gate, Q8_0 weights, 512 tokens); its line carries the time of the
dispatch (histogram, scan, permutation) beside the other stages.
`--workload stack` measures BASELINE config 5: 32 such layers chained on one GPU (26 GB of Q4_K blocks resident),
each y = x + moe(rms_norm(x)), a 32-token batch run for `--steps` (default 128) consecutive steps, each step
feeding the previous output plus N(0, 0.1) noise; a "step" is one pass through all 32 layers.
"""
import argparse
import re
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

H, F, E, TOPK = 4096, 14336, 8, 2
Q4K, Q8_0 = 12, 8
# other weight formats for the decode workload: name -> (GGML dtype, block elements, block bytes, offsets of the f16 scale fields)
FORMATS = {"q4_k": (12, 256, 144, (0, 2)), "q4_0": (2, 32, 18, (0,)), "q4_1": (3, 32, 20, (0, 2)), "q5_0": (6, 32, 22, (0,)),
           "q5_1": (7, 32, 24, (0, 2)), "q8_0": (8, 32, 34, (0,)), "q2_k": (10, 256, 84, (80, 82)), "q3_k": (11, 256, 110, (108,)),
           "q5_k": (13, 256, 176, (0, 2)), "q6_k": (14, 256, 210, (208,))}
CFG4 = dict(H=2048, F=1408, E=60, k=4, Fs=5632)   # BASELINE config 4
EXPERT_BYTES = 3 * H * F * 144 // 256          # 99,090,432 B of Q4_K blocks per expert
HBM_PEAK_GBS = 8000.0                          # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0                        # MI355X dense int8 MFMA, published
# per-expert logit biases under which top-2 routing of N(0, 1.28^2) logits gives Zipf(1) loads (shares 1/i)
ZIPF_BIAS = [0.0, -1.158, -1.581, -1.845, -2.033, -2.186, -2.299, -2.398]


def random_blocks(np, rng, fmt, n_elems):
    """Raw GGML blocks with random payloads; the f16 scale fields are set to 0.001 so that every value is finite."""
    _, be, bb, scale_at = FORMATS[fmt]
    raw = rng.integers(0, 256, (n_elems // be, bb), dtype=np.uint8)
    d = int(np.float16(0.001).view(np.uint16))
    for o in scale_at:
        raw[:, o] = d & 255
        raw[:, o + 1] = d >> 8
    return raw.reshape(-1)


def build_layer(torch, candle_amd, seed=0, gate_bias=None, cfg4=False, fmt="q4_k"):
    """Weights drawn on the GPU, quantised there with the library's QTensor::quantize kernel
    (bit-identical to candle's CPU quantiser), kept as host bytes for the CPU baseline too."""
    h, f, e_n, k, dt, fs = (CFG4["H"], CFG4["F"], CFG4["E"], CFG4["k"], Q8_0, CFG4["Fs"]) if cfg4 else (H, F, E, TOPK, Q4K, 0)
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    if fmt != "q4_k" and not cfg4:
        import numpy as np
        dt = FORMATS[fmt][0]
        rng = np.random.default_rng(seed)

    def draw(shape):
        if fmt != "q4_k" and not cfg4:
            return random_blocks(np, rng, fmt, shape[0] * shape[1])
        x = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * 0.02
        return candle_amd.quantize_weights(dt, x).cpu().numpy()

    w = {"w1": [], "w3": [], "w2": []}
    for e in range(e_n):
        for name, shape in (("w1", (f, h)), ("w3", (f, h)), ("w2", (h, f))):
            w[name].append(draw(shape))
    kw = {}
    if fs:
        w["shared"] = (draw((fs, h)), draw((fs, h)), draw((h, fs)))
    g.manual_seed(seed + 1)
    gate = (torch.randn((e_n, h), generator=g, device="cuda", dtype=torch.float32) * 0.02).cpu().numpy()
    if fs:
        w["shared_gate"] = (torch.randn((h,), generator=g, device="cuda", dtype=torch.float32) * 0.02).cpu().numpy()
        kw = dict(shared_ffn=fs, shared_w1=w["shared"][0], shared_w3=w["shared"][1], shared_w2=w["shared"][2],
                  shared_gate=w["shared_gate"])
    layer = candle_amd.SparseMoeBlock(h, f, e_n, k, dt, gate, w["w1"], w["w3"], w["w2"], gate_bias=gate_bias, **kw)
    return layer, gate, w


def hip_events():
    """HIP events on an explicit stream via ctypes (torch's events only see torch's streams)."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipEventSynchronize.argtypes = [C.c_void_p]
    hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
    return hip


def cpu_baseline(gate, w, xs_host, logits_host, min_seconds, gate_bias=None, cfg4=False, dt=Q4K):
    """candle's CPU path restated (the oracle: serial rows, columns threaded, AVX2 inner loops of
    candle's x86 build) on all host cores: the same batch, same weight bytes, same routing,
    repeated until `min_seconds` of wall time have passed."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import pyoracle as O

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    if cfg4:
        layer = O.Layer(CFG4["H"], CFG4["F"], CFG4["E"], CFG4["k"], Q8_0, gate, w["w1"], w["w3"], w["w2"], Fs=CFG4["Fs"],
                        sw1=w["shared"][0], sw3=w["shared"][1], sw2=w["shared"][2], shared_gate=w["shared_gate"])
    else:
        layer = O.Layer(H, F, E, TOPK, dt, gate, w["w1"], w["w3"], w["w2"], gate_bias=gate_bias)
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


def measured_traffic(batch, name="q4k_up_decode_hbm_traffic.md", key=None):
    """HBM bytes per launch of the up kernel from the committed rocprofv3 counter summary (FETCH_SIZE +
    WRITE_SIZE, scaled by the copy kernel), or None when the summary does not cover this batch size."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", name)
    key = key or "batch=%d" % batch
    try:
        for line in open(path):
            m = re.match(r"traffic_bytes_per_launch\[([^\]]+)\]:\s*(\d+)", line.strip())
            if m and m.group(1) == key:
                return int(m.group(2))
    except OSError:
        pass
    return None


def run_stack(args, np, torch, candle_amd):
    """BASELINE config 5: `--layers` Mixtral-shape MoE layers chained, each with its own resident copy of its
    weights and its own gate; layer l's experts are the drawn eight rotated by l places (timing does not depend on
    the values, and drawing 26 GB of distinct blocks would only lengthen the set-up)."""
    B = args.batch or 32
    _, gate0, w = build_layer(torch, candle_amd)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    layers = []
    for l in range(args.layers):
        r = l % E
        gate = (torch.randn((E, H), generator=g, device="cuda", dtype=torch.float32) * 0.02).cpu().numpy()
        alpha = (1.0 + 0.1 * torch.randn((H,), generator=g, device="cuda", dtype=torch.float32)).cpu().numpy()
        layers.append(candle_amd.SparseMoeBlock(H, F, E, TOPK, Q4K, gate, w["w1"][r:] + w["w1"][:r], w["w3"][r:] + w["w3"][:r],
                                                w["w2"][r:] + w["w2"][:r], rms_alpha=alpha, rms_eps=1e-5))
    x0 = torch.randn((B, H), generator=g, device="cuda", dtype=torch.float32)
    bufs = [torch.empty_like(x0) for _ in range(2)]
    noise, x_next = torch.empty_like(x0), torch.empty_like(x0)

    def step(h):
        for i, layer in enumerate(layers):
            layer.forward(h, out=bufs[i & 1])
            h = bufs[i & 1]
        noise.normal_(0.0, 0.1, generator=g)
        return torch.add(h, noise, out=x_next)   # the next step's input

    stream = torch.cuda.Stream()
    hip = hip_events()
    with torch.cuda.stream(stream):
        h = x0
        for _ in range(args.warmup):
            h = step(h)
        stream.synchronize()
        ev = [C.c_void_p() for _ in range(2)]
        for e in ev:
            hip.hipEventCreate(C.byref(e))
        sh = C.c_void_p(stream.cuda_stream)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        hip.hipEventRecord(ev[0], sh)
        for _ in range(args.steps):
            h = step(h)
        hip.hipEventRecord(ev[1], sh)
        hip.hipEventSynchronize(ev[1])
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms = C.c_float()
        hip.hipEventElapsedTime(C.byref(ms), ev[0], ev[1])
        ms_per_step = ms.value / args.steps
        finite = bool(torch.isfinite(h).all())
        # stage times of a mid-stack layer, measured right after its predecessors ran (its weights and gate are cold)
        mid = len(layers) // 2
        stage = {k: 0.0 for k in layers[mid].STAGES}
        for _ in range(5):
            hh = x0
            for i, layer in enumerate(layers[:mid]):
                layer.forward(hh, out=bufs[i & 1])
                hh = bufs[i & 1]
            for k, v in layers[mid].forward_timed(hh, bufs[mid & 1]).items():
                stage[k] += v / 5
    stage_us = {k: round(v * 1e3, 2) for k, v in stage.items()}
    n_active = E   # a 32-token batch reaches every expert (64 assignments over 8 experts)
    act = 36 / 256
    up_bytes = n_active * (2 * H * F * 144 // 256) + int(B * H * (1 + act)) + int(B * TOPK * F * (1 + act))
    achieved = up_bytes / (stage["up"] * 1e-3) / 1e9
    step_bytes = len(layers) * (n_active * EXPERT_BYTES + E * H * 4 + 3 * B * H * 4)
    out = {
        "metric": "MoE stack tokens/s end to end (%d Mixtral-8x7B MoE layers, Q4_K, decode)" % len(layers),
        "value": B / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8", "data": "synthetic",
        "config": {"workload": "BASELINE config 5: %d chained MoE layers (hidden 4096, ffn 14336, 8 experts, top-2, Q4_K, %.1f GB "
                               "resident), y = x + moe(rms_norm(x)) per layer, %d-token batch, each step fed the previous output "
                               "plus N(0, 0.1) noise" % (len(layers), len(layers) * E * EXPERT_BYTES / 1e9, B),
                   "layers": len(layers), "us_per_layer": ms_per_step * 1e3 / len(layers), "wall_ms_per_step": wall * 1e3 / args.steps,
                   "mid_stack_stage_us": stage_us, "output_finite": finite,
                   "step_algorithmic_bytes": step_bytes, "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "roofline": {"bound": "hbm", "kernel": "q4k_up (w1, w3, SiLU, Q8K re-quantisation), layer %d of the stack" % mid,
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_launch": up_bytes, "launch_us": stage_us["up"]},
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default 200; 128 for the stack workload)")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=None, help="tokens per step (default 32 for decode, 4096 for prefill, 512 for config4)")
    ap.add_argument("--workload", choices=("decode", "prefill", "config4", "stack"), default="decode")
    ap.add_argument("--layers", type=int, default=32, help="layers of the stack workload")
    ap.add_argument("--weights", choices=sorted(FORMATS), default="q4_k", help="GGML format of the expert matrices (decode workload)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--stage-iters", type=int, default=50)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain 1 GiB device copy (the known-size kernel that scales rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE readings) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU only (no collectives, no sharding); --gpus %d is not supported" % args.gpus)

    import numpy as np
    import torch
    import candle_amd

    candle_amd.load_library()  # fails loudly if the HIP extension is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": src.numel() * 4, "copy_bytes_written": src.numel() * 4}))
        return
    if args.steps is None:
        args.steps = 128 if args.workload == "stack" else 200
    if args.workload == "stack":
        if args.weights != "q4_k":
            sys.exit("bench.py: --weights applies to the decode workload only")
        return run_stack(args, np, torch, candle_amd)
    prefill = args.workload == "prefill"
    cfg4 = args.workload == "config4"
    B = args.batch or (4096 if prefill else 512 if cfg4 else 32)
    bias = np.array(ZIPF_BIAS, dtype=np.float32) if prefill else None
    if args.weights != "q4_k" and args.workload != "decode":
        sys.exit("bench.py: --weights applies to the decode workload only")
    layer, gate, w = build_layer(torch, candle_amd, gate_bias=bias, cfg4=cfg4, fmt=args.weights)
    fmt_dt, fmt_be, fmt_bb, _ = FORMATS[args.weights]
    n_exp, hid = (CFG4["E"], CFG4["H"]) if cfg4 else (E, H)
    g = torch.Generator(device="cuda")
    g.manual_seed(2)
    # several distinct activation batches, rotated, so that no step repeats the previous one's input
    xs = [torch.randn((B, hid), generator=g, device="cuda", dtype=torch.float32) for _ in range(4)]
    ys = [torch.empty_like(x) for x in xs]

    stream = torch.cuda.Stream()
    hip = hip_events()
    with torch.cuda.stream(stream):
        for i in range(args.warmup):
            layer.forward(xs[i % 4], out=ys[i % 4])
        stream.synchronize()
        loads = np.diff(layer.last_routing(B)[2])[:n_exp]
        n_active = int((loads > 0).sum())
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

    expert_bytes = 3 * H * F * fmt_bb // fmt_be
    step_bytes = n_active * expert_bytes + E * H * 4 + 2 * B * H * 4
    metric = "MoE layer tokens/s (Mixtral-8x7B shape, Q4_K, %s)" % args.workload
    if cfg4:
        # Weights are Q8_0 (34 bytes per 32 elements); every routed expert with a token and the shared expert are
        # read at least once per step.  The up kernel (w1, w3 of the routed experts) is the longest launch.
        c = CFG4
        expert_bytes = 3 * c["H"] * c["F"] * 34 // 32
        shared_bytes = 3 * c["H"] * c["Fs"] * 34 // 32
        step_bytes = n_active * expert_bytes + shared_bytes + c["E"] * c["H"] * 4 + 2 * B * c["H"] * 4
        up_bytes = n_active * (2 * c["H"] * c["F"] * 34 // 32)
        achieved = up_bytes / (stage["up"] * 1e-3) / 1e9
        step_ops = 2.0 * B * 3 * c["H"] * (c["k"] * c["F"] + c["Fs"])
        roofline = {"bound": "hbm", "kernel": "q32s_up (routed w1, w3, SiLU, Q8_0 re-quantisation; lists beyond 32 rows re-read the weights from L2)",
                    "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                    "traffic": measured_traffic(B, "q32s_config4_kernel_trace.md", "config4") if B == 512 else None,
                    "algorithmic_bytes_per_launch": up_bytes, "launch_us": stage_us["up"]}
        workload = ("BASELINE config 4: hidden 2048, 60 experts of ffn 1408, top-4 renormalised, shared expert of ffn 5632 "
                    "with sigmoid gate, Q8_0 weights, %d tokens" % B)
        extra = {"step_algorithmic_bytes": step_bytes, "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
                 "step_int8_ops": step_ops, "dispatch_us": stage_us["dispatch"], "max_expert_load": int(loads.max())}
        metric = "MoE layer tokens/s (Qwen-MoE shape, Q8_0, 512-token batch)"
    elif prefill:
        # Roofline of the dominant kernel, the tiled up projection: 2 * slots * 2 * H * F integer
        # multiply-adds (w1 and w3) per launch against the dense int8 MFMA peak.
        up_ops = 2.0 * B * TOPK * 2 * H * F
        achieved = up_ops / (stage["up"] * 1e-3) / 1e12
        step_ops = 2.0 * B * TOPK * 3 * H * F
        roofline = {"bound": "mfma", "kernel": "q4k_gemm up (w1, w3, SiLU; int8 MFMA 16x16x64, two scale planes)",
                    "achieved": achieved, "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": achieved / INT8_PEAK_TOPS,
                    "traffic": None, "algorithmic_ops_per_launch": up_ops, "launch_us": stage_us["up"],
                    # every algorithmic multiply-add is issued twice (the 6-bit scale is split over two
                    # pre-scaled int8 planes so that the integer sums stay exact): share of the peak the
                    # MFMA pipe is actually kept busy with, slot tiles padded to 64 / 128 not counted
                    "mfma_issued_frac": 2.0 * achieved / INT8_PEAK_TOPS}
        workload = ("BASELINE config 3: hidden 4096, ffn 14336, 8 experts, top-2, Q4_K weights, prefill of %d tokens, "
                    "Zipf(1) expert load" % B)
        extra = {"expert_loads": [int(v) for v in loads], "step_int8_ops": step_ops,
                 "step_mfma_frac": step_ops / (ms_per_step * 1e-3) / 1e12 / INT8_PEAK_TOPS}
    else:
        # Roofline of the dominant kernel, the up projection (w1, w3 + SiLU): it streams w1 and w3 of
        # every active expert exactly once per launch; algorithmic bytes = Q4_K bytes of those matrices
        # plus the quantised activations it reads and the quantised intermediate it writes.
        act = 36 / 256 if fmt_be == 256 else 8 / 32    # bytes of scales and sums per quantised activation element
        up_bytes = n_active * (2 * H * F * fmt_bb // fmt_be) + int(B * H * (1 + act)) + int(B * TOPK * F * (1 + act))
        achieved = up_bytes / (stage["up"] * 1e-3) / 1e9
        q4k = args.weights == "q4_k"
        roofline = {"bound": "hbm", "kernel": "q4k_up (w1, w3, SiLU, Q8K re-quantisation)" if q4k else "up projection (w1, w3, SiLU, re-quantisation), %s" % args.weights,
                    "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                    "traffic": measured_traffic(B) if q4k else None,
                    "algorithmic_bytes_per_launch": up_bytes, "launch_us": stage_us["up"]}
        workload = "BASELINE config 2: hidden 4096, ffn 14336, 8 experts, top-2, Q4_K weights, decode batch %d" % B
        if not q4k:
            workload = "BASELINE config 2's layer with %s weights (random block payloads), decode batch %d" % (args.weights, B)
            metric = "MoE layer tokens/s (Mixtral-8x7B shape, %s, decode)" % args.weights
        extra = {"step_algorithmic_bytes": step_bytes,
                 "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS}
    out = {
        "metric": metric, "value": tokens_per_s, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8",
        "data": "synthetic",
        "config": dict({"workload": workload, "active_experts": n_active,
                        "wall_ms_per_step": wall * 1e3 / args.steps, "stage_us": stage_us,
                        # a stage that launches nothing still reads what its pair of event records costs
                        "empty_stage_us": min(stage_us.values())}, **extra),
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        layer.forward(xs[0], out=ys[0])
        torch.cuda.synchronize()
        # a bounded sample: the CPU path does ~1 k tokens/s, so a prefill batch is cut to its first 64 tokens
        n_cpu = min(B, 64)
        out["cpu_baseline"] = cpu_baseline(gate, w, xs[0][:n_cpu].cpu().numpy(), layer.last_logits(B)[:n_cpu],
                                           args.cpu_seconds, gate_bias=bias, cfg4=cfg4, dt=fmt_dt)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
