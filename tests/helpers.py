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


class FlipExplainer:
    """Accounts for the outputs of a K-quant layer that lie further from candle's result than the bar.

    The intermediate h = silu(w1 x) * (w3 x) is re-quantised to Q8K before w2 (k_quants.rs:1819-1856).  Two correct
    evaluations that add the f32 partial sums of the first product in different orders differ in h by an ulp here and
    there; where h / d sits on a rounding boundary the quantised value then differs by one step, and the output row of
    that token moves by  (+-1) * routing weight * d_block * dequantised w2[:, j]  -- one column of w2, one quantisation
    step.  candle's own scalar and AVX2 paths differ from each other in this way.  `explain` removes, greedily, up to
    `max_flips` such terms from an error row, each checked to be at most two steps of its block (both evaluations may
    have moved, in opposite directions), and returns what is left: an error that is a wrong term or a wrong index is
    dense in the row and cannot be removed this way."""

    def __init__(self, ref):
        self.ref = ref
        self._w2 = {}

    def w2(self, e):
        if e not in self._w2:
            H, F = self.ref.H, self.ref.F
            W = O.dequantize(self.ref.dtype_down, self.ref.w2[e], H * F).reshape(H, F)
            self._w2[e] = (W, np.einsum("ij,ij->j", W, W, dtype=np.float64))
        return self._w2[e]

    def steps(self, x_row, e, weight):
        """Largest change of an output coefficient that one quantisation step of h[j] makes, per position j."""
        ref = self.ref
        x = np.ascontiguousarray(x_row, dtype=np.float32).reshape(1, -1)
        a = O.matmul(ref.dtype, x, ref.w1[e], ref.F, simd=True)[0]
        b = O.matmul(ref.dtype, x, ref.w3[e], ref.F, simd=True)[0]
        h = (a / (1.0 + np.exp(-a.astype(np.float64))) * b).astype(np.float32)   # a bound on the step: f64 exp will do
        amax = np.abs(h.reshape(-1, 256)).max(axis=1)          # BlockQ8K: d = max / -128
        return np.repeat(amax / 128.0, 256) * abs(float(weight))

    def explain(self, err_row, x_row, experts, weights, bar, max_flips=4):
        """err_row: this path's output row minus candle's (f32 [H]); x_row: the row the experts saw (after the pre-norm);
        experts / weights: the token's routing.  Returns (largest |residual|, [(expert, j, coefficient / step)])."""
        r = np.asarray(err_row, dtype=np.float64).copy()
        found = []
        step = {}
        for _ in range(max_flips):
            if np.abs(r).max() <= bar:
                break
            best = None
            for e, w in zip(experts, weights):
                W, n2 = self.w2(int(e))
                c = (W.T @ r.astype(np.float32)).astype(np.float64) / np.maximum(n2, 1e-300)
                j = int(np.argmax(c * c * n2))
                if best is None or c[j] ** 2 * n2[j] > best[0]:
                    best = (c[j] ** 2 * n2[j], int(e), j, float(c[j]), float(w))
            _, e, j, c, w = best
            if e not in step:
                step[e] = self.steps(x_row, e, w)
            ratio = abs(c) / max(step[e][j], 1e-300)
            if ratio > 2.1:      # more than two quantisation steps at one position: not a flip
                break
            r -= c * self.w2(e)[0][:, j].astype(np.float64)
            found.append((e, j, c / max(step[e][j], 1e-300)))
        return float(np.abs(r).max()), found
