#!/usr/bin/env python3
"""Benchmark of the quantized sparse-MoE block on one MI355X.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|decode|prefill|config4|stack] ...

The line's `value` / `roofline` are BASELINE config 2 at decode batch 32: one Mixtral-8x7B-shape MoE layer (hidden
4096, expert FFN 14336, 8 experts, top-2, Q4_K weights drawn N(0, 0.02) and quantised with candle's algorithm, f32
router gate), N(0, 1) activations already resident in HBM; a "step" is one forward of the layer.  BASELINE's metric names
three quantities (tokens/s; decode HBM share of peak; prefill MFMA share of peak), so the default run (`--workload all`)
measures the other regimes in the same process and reports them as sub-objects of `config`:

  config.prefill  BASELINE config 3: the same layer, 4096 tokens, router bias that makes the expert load follow Zipf(1);
                  tokens/s, the tiled up kernel's int8 TOP/s against the dense int8 MFMA peak, the whole step's share.
  config.cfg4     BASELINE config 4: hidden 2048, 60 experts of FFN 1408, top-4, one always-on shared expert of FFN 5632
                  behind a sigmoid gate, Q8_0 weights, 512 tokens.
  config.stack    BASELINE config 5: 32 such Mixtral layers chained on one GPU (26 GB of Q4_K blocks resident), each
                  y = x + moe(rms_norm(x)), a 32-token batch for 128 consecutive steps, each step fed the previous output
                  plus N(0, 0.1) noise; end-to-end tokens/s.

`--workload decode|prefill|config4|stack` measures one of them alone as the line's `value`.
`--workload prefill [--weights q2_k|q3_k|q5_k|q6_k] [--weights-down q5_k|q6_k]` measures the prefill with Q2_K / Q3_K / Q5_K / Q6_K w1 / w3 and / or w2 stored
in another K-quant (Q4_K_M and Q5_K_M files store part of w2 as Q6_K).
`--weights q4_0|q4_1|q5_0|q5_1|q8_0|q2_k|q3_k|q5_k|q6_k` runs the decode workload on the same layer shape with another
GGML format (random block payloads with small finite scales: timing does not depend on the values).

Timing.  Every measurement first runs forwards for at least 0.5 s (clocks and caches settle; `--warmup` steps are run
on top), then times max(K, 200) steps (decode, config 4) in one region bracketed by HIP events on the launch stream and
host synchronisation: `steps` repeats K as given, `timed_steps` says how many were timed, `ms_per_step` is their mean.
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
MIN_WARM_SECONDS = 0.5
MIN_TIMED_STEPS = 200


def random_blocks(np, rng, fmt, n_elems):
    """Raw GGML blocks with random payloads; the f16 scale fields are set to 0.001 so that every value is finite."""
    _, be, bb, scale_at = FORMATS[fmt]
    raw = rng.integers(0, 256, (n_elems // be, bb), dtype=np.uint8)
    d = int(np.float16(0.001).view(np.uint16))
    for o in scale_at:
        raw[:, o] = d & 255
        raw[:, o + 1] = d >> 8
    return raw.reshape(-1)


def draw_weights(torch, candle_amd, seed=0, cfg4=False, fmt="q4_k", fmt_down=None, quantise=False):
    """Weights drawn on the GPU, quantised there with the library's QTensor::quantize kernel (bit-identical to candle's
    CPU quantiser), returned as host bytes (the CPU baseline runs on the same bytes)."""
    h, f, e_n, dt, fs = (CFG4["H"], CFG4["F"], CFG4["E"], Q8_0, CFG4["Fs"]) if cfg4 else (H, F, E, Q4K, 0)
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    random_payload = fmt != "q4_k" and not cfg4 and not quantise
    if fmt != "q4_k" and not cfg4:
        import numpy as np
        dt = FORMATS[fmt][0]
        rng = np.random.default_rng(seed)

    dt_down = FORMATS[fmt_down][0] if fmt_down else dt

    def draw(shape, dtype=None):
        if random_payload:
            return random_blocks(np, rng, fmt, shape[0] * shape[1])
        x = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * 0.02
        return candle_amd.quantize_weights(dtype or dt, x).cpu().numpy()

    w = {"w1": [], "w3": [], "w2": [], "dt": dt, "dt_down": dt_down}
    for e in range(e_n):
        for name, shape in (("w1", (f, h)), ("w3", (f, h)), ("w2", (h, f))):
            w[name].append(draw(shape, dt_down if name == "w2" else None))
    if fs:
        w["shared"] = (draw((fs, h)), draw((fs, h)), draw((h, fs)))
    g.manual_seed(seed + 1)
    w["gate"] = (torch.randn((e_n, h), generator=g, device="cuda", dtype=torch.float32) * 0.02).cpu().numpy()
    if fs:
        w["shared_gate"] = (torch.randn((h,), generator=g, device="cuda", dtype=torch.float32) * 0.02).cpu().numpy()
    return w


def make_layer(candle_amd, w, gate_bias=None, cfg4=False):
    if cfg4:
        c = CFG4
        return candle_amd.SparseMoeBlock(c["H"], c["F"], c["E"], c["k"], Q8_0, w["gate"], w["w1"], w["w3"], w["w2"], shared_ffn=c["Fs"],
                                         shared_w1=w["shared"][0], shared_w3=w["shared"][1], shared_w2=w["shared"][2], shared_gate=w["shared_gate"])
    return candle_amd.SparseMoeBlock(H, F, E, TOPK, w["dt"], w["gate"], w["w1"], w["w3"], w["w2"], gate_bias=gate_bias,
                                     ggml_dtype_down=w.get("dt_down", w["dt"]))


def hip_events():
    """HIP events on an explicit stream via ctypes (torch's events only see torch's streams)."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipEventSynchronize.argtypes = [C.c_void_p]
    hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
    return hip


class Timer:
    """Times a callable `step(i)` on a torch stream: warm-up by time, then n steps between two HIP events recorded on
    that stream, bracketed by host synchronisation."""

    def __init__(self, torch):
        self.torch = torch
        self.hip = hip_events()
        self.stream = torch.cuda.Stream()
        self.ev = [C.c_void_p() for _ in range(2)]
        for e in self.ev:
            self.hip.hipEventCreate(C.byref(e))

    def run(self, step, n_steps, warmup, min_warm_seconds=MIN_WARM_SECONDS):
        torch = self.torch
        with torch.cuda.stream(self.stream):
            i, t0 = 0, time.perf_counter()
            while i < warmup or time.perf_counter() - t0 < min_warm_seconds:
                step(i)
                i += 1
                if i % 16 == 0:
                    self.stream.synchronize()   # the clock above is the host's: keep it honest
            self.stream.synchronize()
            sh = C.c_void_p(self.stream.cuda_stream)
            torch.cuda.synchronize()
            w0 = time.perf_counter()
            self.hip.hipEventRecord(self.ev[0], sh)
            for j in range(n_steps):
                step(i + j)
            self.hip.hipEventRecord(self.ev[1], sh)
            self.hip.hipEventSynchronize(self.ev[1])
            torch.cuda.synchronize()
            wall = time.perf_counter() - w0
            ms = C.c_float()
            self.hip.hipEventElapsedTime(C.byref(ms), self.ev[0], self.ev[1])
        return ms.value / n_steps, wall * 1e3 / n_steps, i

    def stages(self, layer, xs, ys, iters):
        """Per-stage durations: HIP events recorded by the library between its launches, on this stream."""
        stage = {k: 0.0 for k in layer.STAGES}
        with self.torch.cuda.stream(self.stream):
            for i in range(iters):
                for k, v in layer.forward_timed(xs[i % len(xs)], ys[i % len(ys)]).items():
                    stage[k] += v / iters
        return stage


def cpu_baseline(w, xs_host, logits_host, min_seconds, gate_bias=None, cfg4=False):
    """candle's CPU path restated (the oracle: serial rows, columns threaded, AVX2 inner loops of candle's x86 build) on
    all host cores: the same batch, same weight bytes, same routing, repeated until `min_seconds` of wall time have passed."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import pyoracle as O

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    if cfg4:
        layer = O.Layer(CFG4["H"], CFG4["F"], CFG4["E"], CFG4["k"], Q8_0, w["gate"], w["w1"], w["w3"], w["w2"], Fs=CFG4["Fs"],
                        sw1=w["shared"][0], sw3=w["shared"][1], sw2=w["shared"][2], shared_gate=w["shared_gate"])
    else:
        layer = O.Layer(H, F, E, TOPK, w["dt"], w["gate"], w["w1"], w["w3"], w["w2"], gate_bias=gate_bias, dtype_down=w.get("dt_down", w["dt"]))
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


def profile_build_id(name):
    """The `library_build_id: <id>` line of a committed profile summary: the sources the profiled library was built from."""
    try:
        for line in open(os.path.join(ROOT, "profiles", name)):
            m = re.match(r"library_build_id:\s*([0-9a-f]+)", line.strip())
            if m:
                return m.group(1)
    except OSError:
        pass
    return None


def counter_figure(name, label, key):
    """(value, note) for a `label[key]: value` line of a committed rocprofv3 counter summary.  Such a figure belongs to
    the build it was measured on: it is given only when the summary's recorded build id equals the loaded library's
    (moe_build_id); otherwise the value is None and the note says which ids differ.  Never a reading of this run."""
    import candle_amd
    lib_id, prof_id = candle_amd.build_id(), profile_build_id(name)
    if prof_id != lib_id:
        return None, "profiles/%s was measured on build %s, the loaded library is build %s: figure withheld" % (name, prof_id, lib_id)
    try:
        for line in open(os.path.join(ROOT, "profiles", name)):
            m = re.match(r"%s\[([^\]]+)\]:\s*([0-9.eE+-]+)" % re.escape(label), line.strip())
            if m and m.group(1) == key:
                v = float(m.group(2))
                return (int(v) if v == int(v) and "." not in m.group(2) else v), \
                    "profiles/%s (committed rocprofv3 --pmc summary of build %s, the build loaded now; not a reading of this run)" % (name, prof_id)
    except OSError:
        pass
    return None, "profiles/%s holds no %s[%s]" % (name, label, key)


def activations(torch, B, hid, seed=2, n=4):
    """Several distinct activation batches, rotated, so that no step repeats the previous one's input."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    xs = [torch.randn((B, hid), generator=g, device="cuda", dtype=torch.float32) for _ in range(n)]
    return xs, [torch.empty_like(x) for x in xs]


def measure_decode(args, np, torch, timer, layer, B, fmt="q4_k"):
    xs, ys = activations(torch, B, H)
    n_steps = max(args.steps, MIN_TIMED_STEPS)
    ms, wall_ms, warmed = timer.run(lambda i: layer.forward(xs[i % 4], out=ys[i % 4]), n_steps, args.warmup)
    loads = np.diff(layer.last_routing(B)[2])[:E]
    n_active = int((loads > 0).sum())
    stage = timer.stages(layer, xs, ys, args.stage_iters)
    stage_us = {k: round(v * 1e3, 2) for k, v in stage.items()}
    fmt_dt, fmt_be, fmt_bb, _ = FORMATS[fmt]
    expert_bytes = 3 * H * F * fmt_bb // fmt_be
    step_bytes = n_active * expert_bytes + E * H * 4 + 2 * B * H * 4
    # Roofline of the dominant kernel, the up projection (w1, w3 + SiLU): it streams w1 and w3 of every active expert
    # exactly once per launch; algorithmic bytes = the blocks of those matrices plus the quantised activations it reads
    # and the quantised intermediate it writes.
    act = 36 / 256 if fmt_be == 256 else 8 / 32    # bytes of scales and sums per quantised activation element
    up_bytes = n_active * (2 * H * F * fmt_bb // fmt_be) + int(B * H * (1 + act)) + int(B * TOPK * F * (1 + act))
    achieved = up_bytes / (stage["up"] * 1e-3) / 1e9
    q4k = fmt == "q4_k"
    traffic, traffic_note = counter_figure("q4k_up_decode_hbm_traffic.md", "traffic_bytes_per_launch", "batch=%d" % B) if q4k else (None, None)
    roofline = {"bound": "hbm", "kernel": "q4k_up (w1, w3, SiLU, Q8K re-quantisation)" if q4k else "up projection (w1, w3, SiLU, re-quantisation), %s" % fmt,
                "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                "traffic_source": traffic_note,
                "algorithmic_bytes_per_launch": up_bytes, "launch_us": stage_us["up"]}
    return {"tokens_per_s": B / (ms * 1e-3), "ms_per_step": ms, "wall_ms_per_step": wall_ms, "timed_steps": n_steps, "warmup_steps_run": warmed,
            "batch": B, "active_experts": n_active, "stage_us": stage_us, "empty_stage_us": min(stage_us.values()),
            "step_algorithmic_bytes": step_bytes, "step_hbm_frac": step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "roofline": roofline, "xs": xs, "ys": ys}


def measure_decode_batches(args, np, torch, timer, layer, batches=(1, 8, 64)):
    """The other batch sizes BASELINE config 2 names, briefly (200 timed steps each): step time and the share of the HBM
    peak the step's algorithmic bytes reach.  Batch 1 also as a HIP graph of four forwards (the four rotating inputs,
    whose routings differ) replayed back to back: what the step takes without the host's launch gaps."""
    out = []
    for B in batches:
        xs, ys = activations(torch, B, H)
        ms, _, _ = timer.run(lambda i: layer.forward(xs[i % 4], out=ys[i % 4]), MIN_TIMED_STEPS, 10, min_warm_seconds=0.3)
        active = []
        for i in range(4):   # the four inputs select different experts: bytes are those of their mean
            layer.forward(xs[i], out=ys[i])
            active.append(int((np.diff(layer.last_routing(B)[2])[:E] > 0).sum()))
        n_active = sum(active) / 4.0
        step_bytes = n_active * EXPERT_BYTES + E * H * 4 + 2 * B * H * 4
        rec = {"batch": B, "active_experts": n_active, "us_per_step": ms * 1e3, "tokens_per_s": B / (ms * 1e-3),
               "step_algorithmic_bytes": step_bytes, "step_hbm_frac": step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        if B == 1:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=timer.stream):
                for i in range(4):
                    layer.forward(xs[i], out=ys[i])
            g_ms, _, _ = timer.run(lambda i: graph.replay(), 50, 5, min_warm_seconds=0.2)
            rec["graph_us_per_step"] = g_ms * 1e3 / 4
            rec["graph_step_hbm_frac"] = step_bytes / (g_ms * 1e-3 / 4) / 1e9 / HBM_PEAK_GBS
            del graph
        out.append(rec)
    return out


def measure_prefill(args, np, torch, timer, layer, B):
    xs, ys = activations(torch, B, H, n=2)
    n_steps = max(20, min(args.steps, 50))
    ms, wall_ms, warmed = timer.run(lambda i: layer.forward(xs[i % 2], out=ys[i % 2]), n_steps, min(args.warmup, 5))
    loads = np.diff(layer.last_routing(B)[2])[:E]
    stage = timer.stages(layer, xs, ys, max(3, min(args.stage_iters, 10)))
    stage_us = {k: round(v * 1e3, 2) for k, v in stage.items()}
    # Roofline of the dominant kernel, the tiled up projection: 2 * slots * 2 * H * F integer multiply-adds (w1 and w3)
    # per launch against the dense int8 MFMA peak.
    up_ops = 2.0 * B * TOPK * 2 * H * F
    achieved = up_ops / (stage["up"] * 1e-3) / 1e12
    step_ops = 2.0 * B * TOPK * 3 * H * F
    one_plane = args.weights == "q2_k"   # a 4-bit scale times a 2-bit code fits a byte: one plane, every multiply-add issued once
    q4k = args.weights == "q4_k"
    busy, busy_note = counter_figure("q4k_gemm_prefill_4096_kernel_trace.md", "mfma_busy_frac", "prefill_up") if B == 4096 and q4k else (None, None)
    roofline = {"bound": "mfma", "kernel": "q4k_gemm up (w1, w3, SiLU; int8 MFMA 16x16x64, %s)" % ("one plane of scaled codes" if one_plane else "two scale planes"),
                "achieved": achieved, "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": achieved / INT8_PEAK_TOPS,
                "traffic": None, "algorithmic_ops_per_launch": up_ops, "launch_us": stage_us["up"],
                # every algorithmic multiply-add is issued twice (the 6-bit scale is split over two pre-scaled int8
                # planes so that the integer sums stay exact): share of the peak the MFMA pipe is actually kept busy
                # with, slot tiles padded to 64 / 128 not counted
                "mfma_issued_frac": (1.0 if one_plane else 2.0) * achieved / INT8_PEAK_TOPS,
                # share of the cycles the matrix pipe is busy (SQ_VALU_MFMA_BUSY_CYCLES over the kernel's SIMD cycles)
                # as the committed rocprofv3 counter summary gives it: a figure of that profile, not a reading of this run
                "mfma_pipe_busy_frac": busy, "mfma_pipe_busy_source": busy_note}
    return {"tokens_per_s": B / (ms * 1e-3), "ms_per_step": ms, "wall_ms_per_step": wall_ms, "timed_steps": n_steps, "warmup_steps_run": warmed,
            "tokens": B, "expert_loads": [int(v) for v in loads], "stage_us": stage_us, "step_int8_ops": step_ops,
            "step_mfma_frac": step_ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, "roofline": roofline, "xs": xs, "ys": ys}


def measure_cfg4(args, np, torch, timer, layer, B):
    c = CFG4
    xs, ys = activations(torch, B, c["H"])
    n_steps = max(args.steps, MIN_TIMED_STEPS)
    ms, wall_ms, warmed = timer.run(lambda i: layer.forward(xs[i % 4], out=ys[i % 4]), n_steps, args.warmup)
    loads = np.diff(layer.last_routing(B)[2])[:c["E"]]
    n_active = int((loads > 0).sum())
    stage = timer.stages(layer, xs, ys, args.stage_iters)
    stage_us = {k: round(v * 1e3, 2) for k, v in stage.items()}
    # Weights are Q8_0 (34 bytes per 32 elements); every routed expert with a token and the shared expert are read at
    # least once per step.  The up kernel (w1, w3 of the routed experts) is the longest launch.
    expert_bytes = 3 * c["H"] * c["F"] * 34 // 32
    shared_bytes = 3 * c["H"] * c["Fs"] * 34 // 32
    step_bytes = n_active * expert_bytes + shared_bytes + c["E"] * c["H"] * 4 + 2 * B * c["H"] * 4
    up_bytes = n_active * (2 * c["H"] * c["F"] * 34 // 32)
    achieved = up_bytes / (stage["up"] * 1e-3) / 1e9
    traffic, traffic_note = counter_figure("q8_0_gemm_config4_kernel_trace.md", "traffic_bytes_per_launch", "config4") if B == 512 else (None, None)
    roofline = {"bound": "hbm", "kernel": "q8_0_gemm<0>: routed up projection (w1, w3, SiLU, Q8_0 re-quantisation), 64-slot tiles",
                "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                "traffic_source": traffic_note,
                "algorithmic_bytes_per_launch": up_bytes, "launch_us": stage_us["up"]}
    return {"tokens_per_s": B / (ms * 1e-3), "ms_per_step": ms, "wall_ms_per_step": wall_ms, "timed_steps": n_steps, "warmup_steps_run": warmed,
            "tokens": B, "active_experts": n_active, "max_expert_load": int(loads.max()), "stage_us": stage_us, "dispatch_us": stage_us["dispatch"],
            "step_algorithmic_bytes": step_bytes, "step_hbm_frac": step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "step_int8_ops": 2.0 * B * 3 * c["H"] * (c["k"] * c["F"] + c["Fs"]), "roofline": roofline, "xs": xs, "ys": ys}


def measure_stack(args, np, torch, candle_amd, timer, w, n_layers, n_steps, B=32):
    """BASELINE config 5: `n_layers` Mixtral-shape MoE layers chained, each with its own resident copy of its weights and its
    own gate; layer l's experts are the drawn eight rotated by l places (timing does not depend on the values, and drawing
    26 GB of distinct blocks would only lengthen the set-up)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    layers = []
    for l in range(n_layers):
        r = l % E
        gate = (torch.randn((E, H), generator=g, device="cuda", dtype=torch.float32) * 0.02).cpu().numpy()
        alpha = (1.0 + 0.1 * torch.randn((H,), generator=g, device="cuda", dtype=torch.float32)).cpu().numpy()
        layers.append(candle_amd.SparseMoeBlock(H, F, E, TOPK, Q4K, gate, w["w1"][r:] + w["w1"][:r], w["w3"][r:] + w["w3"][:r],
                                                w["w2"][r:] + w["w2"][:r], rms_alpha=alpha, rms_eps=1e-5))
    x0 = torch.randn((B, H), generator=g, device="cuda", dtype=torch.float32)
    bufs = [torch.empty_like(x0) for _ in range(2)]
    noise, state = torch.empty_like(x0), {"h": x0}
    x_next = torch.empty_like(x0)

    def step(_):
        # one call for the 32 layers (moe_stack_forward_device): a layer's combine pass + residual and the next layer's
        # rms-norm / router / quantiser are one launch
        h = candle_amd.stack_forward(layers, state["h"], out=bufs[0])
        noise.normal_(0.0, 0.1, generator=g)
        state["h"] = torch.add(h, noise, out=x_next)   # the next step's input

    def step_layer_by_layer(_):
        h = state["h"]
        for i, layer in enumerate(layers):
            layer.forward(h, out=bufs[i & 1])
            h = bufs[i & 1]
        noise.normal_(0.0, 0.1, generator=g)
        state["h"] = torch.add(h, noise, out=x_next)

    # the same stack as 32 calls of moe_layer_forward_device, for comparison (--stack-entry-only leaves it out, so that a
    # kernel trace of the run holds the one-call path's launches only)
    lbl_ms = None
    if not args.stack_entry_only:
        lbl_ms, _, _ = timer.run(step_layer_by_layer, 32, 2, min_warm_seconds=0.2)
    state["h"] = x0
    ms, wall_ms, warmed = timer.run(step, n_steps, min(args.warmup, 3), min_warm_seconds=0.3)
    finite = bool(torch.isfinite(state["h"]).all())
    # stage times of a mid-stack layer, measured right after its predecessors ran (its weights and gate are cold)
    mid = len(layers) // 2
    stage = {k: 0.0 for k in layers[mid].STAGES}
    with torch.cuda.stream(timer.stream):
        for _ in range(0 if args.stack_entry_only else 5):
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
    achieved = up_bytes / (stage["up"] * 1e-3) / 1e9 if stage["up"] else 0.0
    step_bytes = len(layers) * (n_active * EXPERT_BYTES + E * H * 4 + 3 * B * H * 4)
    for layer in layers:
        layer.close()
    return {"tokens_per_s": B / (ms * 1e-3), "ms_per_step": ms, "wall_ms_per_step": wall_ms, "timed_steps": n_steps, "warmup_steps_run": warmed,
            "layers": n_layers, "batch": B, "resident_gb": n_layers * E * EXPERT_BYTES / 1e9, "us_per_layer": ms * 1e3 / n_layers,
            "entry": "moe_stack_forward_device (one call per step)", "layer_by_layer_ms_per_step": lbl_ms,
            "mid_stack_stage_us": stage_us, "output_finite": finite, "step_algorithmic_bytes": step_bytes,
            "step_hbm_frac": step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "roofline": {"bound": "hbm", "kernel": "q4k_up (w1, w3, SiLU, Q8K re-quantisation), layer %d of the stack" % mid,
                         "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                         "algorithmic_bytes_per_launch": up_bytes, "launch_us": stage_us["up"]}}


def sub(m):
    """A measurement as a sub-object of `config`: everything but the tensors."""
    return {k: v for k, v in m.items() if k not in ("xs", "ys")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200, help="timed steps K (at least 200 are timed; the stack times its own 128)")
    ap.add_argument("--warmup", type=int, default=20, help="warm-up steps, on top of the 0.5 s every measurement warms up for")
    ap.add_argument("--batch", type=int, default=None, help="tokens per step (default 32 for decode, 4096 for prefill, 512 for config4)")
    ap.add_argument("--workload", choices=("all", "decode", "prefill", "config4", "stack"), default="all")
    ap.add_argument("--layers", type=int, default=32, help="layers of the stack workload")
    ap.add_argument("--stack-steps", type=int, default=128, help="consecutive steps of the stack workload")
    ap.add_argument("--weights", choices=sorted(FORMATS), default="q4_k", help="GGML format of the expert matrices (decode workload)")
    ap.add_argument("--weights-down", choices=("q5_k", "q6_k"), default=None,
                    help="prefill workload: w2 in this format beside the w1 / w3 of --weights (Q4_K_M and Q5_K_M files store part of w2 as Q6_K)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--stage-iters", type=int, default=50)
    ap.add_argument("--stack-entry-only", action="store_true",
                    help="stack workload: skip the layer-by-layer comparison run and the per-stage timing of layer 16")
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
    wl = args.workload
    if args.weights != "q4_k" and wl not in ("decode", "all") and not (wl == "prefill" and args.weights in ("q2_k", "q3_k", "q5_k", "q6_k")):
        sys.exit("bench.py: --weights applies to the decode workload (and the other K-quants to the prefill workload) only")
    if args.weights != "q4_k" and wl != "prefill":
        wl = "decode"
    if args.weights_down and wl != "prefill":
        sys.exit("bench.py: --weights-down applies to the prefill workload only")
    timer = Timer(torch)
    out = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "i8", "data": "synthetic", "unit": "tokens/s", "library_build_id": candle_amd.build_id()}
    bias = np.array(ZIPF_BIAS, dtype=np.float32)
    cpu = None

    if wl == "config4":
        w4 = draw_weights(torch, candle_amd, cfg4=True)
        layer = make_layer(candle_amd, w4, cfg4=True)
        B = args.batch or 512
        m = measure_cfg4(args, np, torch, timer, layer, B)
        out.update(metric="MoE layer tokens/s (Qwen-MoE shape, Q8_0, 512-token batch)", value=m["tokens_per_s"], ms_per_step=m["ms_per_step"],
                   timed_steps=m["timed_steps"], roofline=m["roofline"],
                   config=dict({"workload": "BASELINE config 4: hidden 2048, 60 experts of ffn 1408, top-4 renormalised, shared expert of ffn 5632 "
                                            "with sigmoid gate, Q8_0 weights, %d tokens" % B}, **{k: v for k, v in sub(m).items() if k != "roofline"}))
        if not args.no_cpu_baseline:
            n_cpu = min(B, 64)
            layer.forward(m["xs"][0], out=m["ys"][0])
            torch.cuda.synchronize()
            cpu = cpu_baseline(w4, m["xs"][0][:n_cpu].cpu().numpy(), layer.last_logits(B)[:n_cpu], args.cpu_seconds, cfg4=True)
    elif wl == "stack":
        w = draw_weights(torch, candle_amd)
        m = measure_stack(args, np, torch, candle_amd, timer, w, args.layers, args.stack_steps, args.batch or 32)
        out.update(metric="MoE stack tokens/s end to end (%d Mixtral-8x7B MoE layers, Q4_K, decode)" % args.layers, value=m["tokens_per_s"],
                   ms_per_step=m["ms_per_step"], timed_steps=m["timed_steps"], roofline=m["roofline"],
                   config=dict({"workload": "BASELINE config 5: %d chained MoE layers (hidden 4096, ffn 14336, 8 experts, top-2, Q4_K, %.1f GB resident), "
                                            "y = x + moe(rms_norm(x)) per layer, %d-token batch, each step fed the previous output plus N(0, 0.1) noise"
                                            % (args.layers, m["resident_gb"], m["batch"])}, **{k: v for k, v in m.items() if k != "roofline"}))
    elif wl == "prefill":
        w = draw_weights(torch, candle_amd, fmt=args.weights, fmt_down=args.weights_down, quantise=True)
        layer = make_layer(candle_amd, w, gate_bias=bias)
        B = args.batch or 4096
        m = measure_prefill(args, np, torch, timer, layer, B)
        wdesc = "%s weights" % args.weights if not args.weights_down else "%s w1 / w3 with %s w2" % (args.weights, args.weights_down)
        out.update(metric="MoE layer tokens/s (Mixtral-8x7B shape, Q4_K, prefill)", value=m["tokens_per_s"], ms_per_step=m["ms_per_step"],
                   timed_steps=m["timed_steps"], roofline=m["roofline"],
                   config=dict({"workload": "BASELINE config 3: hidden 4096, ffn 14336, 8 experts, top-2, %s, prefill of %d tokens, "
                                            "Zipf(1) expert load" % (wdesc, B)}, **{k: v for k, v in sub(m).items() if k != "roofline"}))
        if not args.no_cpu_baseline:
            n_cpu = min(B, 64)   # a bounded sample: the CPU path does ~1 k tokens/s
            cpu = cpu_baseline(w, m["xs"][0][:n_cpu].cpu().numpy(), layer.last_logits(B)[:n_cpu], args.cpu_seconds, gate_bias=bias)
    else:
        fmt = args.weights
        w = draw_weights(torch, candle_amd, fmt=fmt)
        layer = make_layer(candle_amd, w)
        B = args.batch or 32
        m = measure_decode(args, np, torch, timer, layer, B, fmt)
        q4k = fmt == "q4_k"
        workload = "BASELINE config 2: hidden 4096, ffn 14336, 8 experts, top-2, Q4_K weights, decode batch %d" % B
        metric = "MoE layer tokens/s (Mixtral-8x7B shape, Q4_K, decode)"
        if not q4k:
            workload = "BASELINE config 2's layer with %s weights (random block payloads), decode batch %d" % (fmt, B)
            metric = "MoE layer tokens/s (Mixtral-8x7B shape, %s, decode)" % fmt
        cfg = dict({"workload": workload}, **{k: v for k, v in sub(m).items() if k != "roofline"})
        out.update(metric=metric, value=m["tokens_per_s"], ms_per_step=m["ms_per_step"], timed_steps=m["timed_steps"], roofline=m["roofline"], config=cfg)
        if not args.no_cpu_baseline:
            layer.forward(m["xs"][0], out=m["ys"][0])
            torch.cuda.synchronize()
            cpu = cpu_baseline(w, m["xs"][0].cpu().numpy(), layer.last_logits(B), args.cpu_seconds)
        if wl == "all" or (wl == "decode" and q4k and args.batch is None):
            # the other batch sizes of BASELINE config 2, on the same layer
            cfg["decode_batches"] = measure_decode_batches(args, np, torch, timer, layer)
        if wl == "all":
            out["metric"] = "MoE layer tokens/s; decode HBM GB/s %peak; prefill MFMA util, Mixtral-8x7B Q4_K"
            # prefill on the same weights, with the router bias that skews the load
            pl = make_layer(candle_amd, w, gate_bias=bias)
            mp = measure_prefill(args, np, torch, timer, pl, 4096)
            cfg["prefill"] = dict({"workload": "BASELINE config 3: the same layer, prefill of 4096 tokens, Zipf(1) expert load"}, **sub(mp))
            pl.close()
            del mp
            w4 = draw_weights(torch, candle_amd, cfg4=True)
            l4 = make_layer(candle_amd, w4, cfg4=True)
            m4 = measure_cfg4(args, np, torch, timer, l4, 512)
            cfg["cfg4"] = dict({"workload": "BASELINE config 4: hidden 2048, 60 experts of ffn 1408, top-4, shared expert of ffn 5632, Q8_0, 512 tokens"}, **sub(m4))
            l4.close()
            del m4, w4
            layer.close()
            ms_ = measure_stack(args, np, torch, candle_amd, timer, w, args.layers, args.stack_steps)
            cfg["stack"] = dict({"workload": "BASELINE config 5: %d chained layers, y = x + moe(rms_norm(x)), 32-token batch, %d steps"
                                             % (args.layers, args.stack_steps)}, **ms_)
            # the three quantities the metric names, side by side
            cfg["summary"] = {"decode_tokens_per_s": m["tokens_per_s"], "decode_step_hbm_frac": m["step_hbm_frac"],
                              "decode_up_kernel_hbm_frac": m["roofline"]["frac"], "prefill_tokens_per_s": cfg["prefill"]["tokens_per_s"],
                              "prefill_up_kernel_int8_frac": cfg["prefill"]["roofline"]["frac"], "prefill_step_int8_frac": cfg["prefill"]["step_mfma_frac"],
                              "cfg4_tokens_per_s": cfg["cfg4"]["tokens_per_s"], "stack_tokens_per_s": cfg["stack"]["tokens_per_s"]}
    if cpu is not None:
        out["cpu_baseline"] = cpu
    print(json.dumps(out))


if __name__ == "__main__":
    main()
