"""Shared builders for the parity tests: one set of seeded weights handed, byte for byte, to both
the CPU oracle and the HIP library."""
import numpy as np

import pyoracle as O

CONFIGS = {
    # BASELINE configs (name -> H, F, E, k, dtype, extras)
    "cfg1": dict(H=1024, F=3584, E=8, k=2, dt=O.Q4_0),
    "cfg2": dict(H=4096, F=14336, E=8, k=2, dt=O.Q4K),
    "cfg4": dict(H=2048, F=1408, E=60, k=4, dt=O.Q8_0, Fs=5632),
}


def make_weights(H, F, E, dt, seed=0, Fs=0, std=0.02, threads=8, dt_down=None):
    """Expert weights N(0, std) quantised by the oracle's quantiser (stream order e, then w1, w3, w2).
    dt_down: dtype of the w2 matrices when it differs from dt."""
    dtd = dt if dt_down is None else dt_down
    w1, w3, w2 = [], [], []
    s = seed * 1000003
    for e in range(E):
        w1.append(O.fill_normal_quantized(s + 3 * e + 0, dt, F, H, std, threads))
        w3.append(O.fill_normal_quantized(s + 3 * e + 1, dt, F, H, std, threads))
        w2.append(O.fill_normal_quantized(s + 3 * e + 2, dtd, H, F, std, threads))
    shared = None
    if Fs:
        shared = (O.fill_normal_quantized(s + 3 * E + 0, dt, Fs, H, std, threads),
                  O.fill_normal_quantized(s + 3 * E + 1, dt, Fs, H, std, threads),
                  O.fill_normal_quantized(s + 3 * E + 2, dtd, H, Fs, std, threads))
    return w1, w3, w2, shared


def make_pair(H, F, E, k, dt, seed=0, Fs=0, rms=False, norm_topk=True, gate_bias=None, want_gpu=True, dt_down=None):
    """Returns (oracle Layer, HIP SparseMoeBlock or None) built from identical bytes."""
    w1, w3, w2, shared = make_weights(H, F, E, dt, seed, Fs, dt_down=dt_down)
    gate = O.fill_normal(seed * 1000003 + 777, E * H, 0.0, 0.02).reshape(E, H)
    kw = dict(norm_topk=norm_topk, gate_bias=gate_bias)
    okw, gkw = dict(kw, dtype_down=dt_down), dict(kw, ggml_dtype_down=dt_down)
    if Fs:
        sg = O.fill_normal(seed * 1000003 + 778, H, 0.0, 0.02)
        okw.update(Fs=Fs, sw1=shared[0], sw3=shared[1], sw2=shared[2], shared_gate=sg)
        gkw.update(shared_ffn=Fs, shared_w1=shared[0], shared_w3=shared[1], shared_w2=shared[2], shared_gate=sg)
    if rms:
        alpha = (1.0 + 0.1 * O.fill_normal(seed * 1000003 + 779, H)).astype(np.float32)
        okw.update(rms_alpha=alpha, rms_eps=1e-5)
        gkw.update(rms_alpha=alpha, rms_eps=1e-5)
    ref = O.Layer(H, F, E, k, dt, gate, w1, w3, w2, **okw)
    gpu = None
    if want_gpu:
        import candle_amd
        gpu = candle_amd.SparseMoeBlock(H, F, E, k, dt, gate, w1, w3, w2, **gkw)
    return ref, gpu


def activations(T, H, seed=2):
    return O.fill_normal(seed * 7919 + 13, T * H, 0.0, 1.0).reshape(T, H)


def rms(a):
    return float(np.sqrt(np.mean(np.asarray(a, dtype=np.float64) ** 2)))
