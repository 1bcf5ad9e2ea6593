"""ctypes front end of the CPU oracle (oracle/libmoe_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke`` and by the
``cpu_baseline`` leg of ``bench.py``; the shipped package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmoe_oracle.so")

Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2K, Q3K, Q4K, Q5K, Q6K, Q8K = 2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15
BLOCK_ELEMS = {Q4_0: 32, Q4_1: 32, Q5_0: 32, Q5_1: 32, Q8_0: 32, Q8_1: 32,
               Q2K: 256, Q3K: 256, Q4K: 256, Q5K: 256, Q6K: 256, Q8K: 256}
BLOCK_BYTES = {Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_0: 34, Q8_1: 36,
               Q2K: 84, Q3K: 110, Q4K: 144, Q5K: 176, Q6K: 210, Q8K: 292}
VECDOT = {Q4_0: Q8_0, Q5_0: Q8_0, Q8_0: Q8_0, Q4_1: Q8_1, Q5_1: Q8_1, Q8_1: Q8_1,
          Q2K: Q8K, Q3K: Q8K, Q4K: Q8K, Q5K: Q8K, Q6K: Q8K, Q8K: Q8K}


def build(force=False):
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force:
        subprocess.run(["make", "-C", HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", HERE], check=True, capture_output=True)


class _Layer(C.Structure):
    _fields_ = [
        ("H", C.c_int64), ("F", C.c_int64), ("E", C.c_int64), ("k", C.c_int64),
        ("dtype", C.c_int), ("norm_topk", C.c_int),
        ("gate", C.c_void_p), ("gate_bias", C.c_void_p),
        ("w1", C.POINTER(C.c_void_p)), ("w3", C.POINTER(C.c_void_p)), ("w2", C.POINTER(C.c_void_p)),
        ("Fs", C.c_int64), ("sw1", C.c_void_p), ("sw3", C.c_void_p), ("sw2", C.c_void_p),
        ("shared_gate", C.c_void_p), ("rms_alpha", C.c_void_p), ("rms_eps", C.c_float),
        ("dtype_down", C.c_int),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_quantize.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]
        L.orc_dequantize.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]
        L.orc_vec_dot.restype = C.c_float
        L.orc_vec_dot.argtypes = [C.c_int, C.c_int64, C.c_void_p, C.c_void_p]
        L.orc_vec_dot_avx2.restype = C.c_float
        L.orc_vec_dot_avx2.argtypes = [C.c_int, C.c_int64, C.c_void_p, C.c_void_p]
        L.orc_matmul.argtypes = [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p,
                                 C.c_void_p, C.c_int, C.c_int]
        L.orc_softmax_last_dim.restype = None
        L.orc_softmax_last_dim.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
        L.orc_silu.restype = C.c_float
        L.orc_silu.argtypes = [C.c_float]
        L.orc_sigmoid.restype = C.c_float
        L.orc_sigmoid.argtypes = [C.c_float]
        L.orc_rms_norm.restype = None
        L.orc_rms_norm.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_float, C.c_void_p]
        L.orc_gate_logits.restype = None
        L.orc_gate_logits.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p]
        L.orc_route.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int] + [C.c_void_p] * 5
        L.orc_moe_forward.argtypes = [C.POINTER(_Layer), C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_int, C.c_int]
        L.orc_fill_normal.restype = None
        L.orc_fill_normal.argtypes = [C.c_uint64, C.c_int64, C.c_float, C.c_float, C.c_void_p, C.c_int]
        L.orc_fill_normal_quantized.argtypes = [C.c_uint64, C.c_int, C.c_int64, C.c_int64, C.c_float,
                                                C.c_void_p, C.c_int]
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def f16_to_f32(h):
    return float(lib().orc_f16_to_f32(int(h)))


def f32_to_f16(f):
    return int(lib().orc_f32_to_f16(float(f)))


def nbytes(dtype, n):
    assert n % BLOCK_ELEMS[dtype] == 0
    return n // BLOCK_ELEMS[dtype] * BLOCK_BYTES[dtype]


def quantize(dtype, x):
    """f32 array (any shape, last dim multiple of the block) -> uint8 array of raw blocks."""
    x = _f32(x)
    out = np.zeros(nbytes(dtype, x.size), dtype=np.uint8)
    if x.ndim > 1:
        assert x.shape[-1] % BLOCK_ELEMS[dtype] == 0
    assert lib().orc_quantize(dtype, _p(x), x.size, _p(out)) == 0
    return out


def dequantize(dtype, blocks, n):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    assert blocks.size == nbytes(dtype, n)
    out = np.empty(n, dtype=np.float32)
    assert lib().orc_dequantize(dtype, _p(blocks), n, _p(out)) == 0
    return out


def vec_dot(dtype, n, w, a, simd=False):
    w = np.ascontiguousarray(w, dtype=np.uint8)
    a = np.ascontiguousarray(a, dtype=np.uint8)
    f = lib().orc_vec_dot_avx2 if simd else lib().orc_vec_dot
    return float(f(dtype, n, _p(w), _p(a)))


def matmul(dtype, lhs, rhs_blocks, n, simd=False, threads=1):
    """lhs [m,k] f32, rhs_blocks = raw blocks of the [n,k] weight -> [m,n] f32."""
    lhs = _f32(lhs)
    m, k = lhs.shape
    rhs_blocks = np.ascontiguousarray(rhs_blocks, dtype=np.uint8)
    assert rhs_blocks.size == nbytes(dtype, n * k)
    dst = np.empty((m, n), dtype=np.float32)
    assert lib().orc_matmul(dtype, m, k, n, _p(lhs), _p(rhs_blocks), _p(dst), int(simd), threads) == 0
    return dst


def softmax_last_dim(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_softmax_last_dim(_p(x), x.size // x.shape[-1], x.shape[-1], _p(y))
    return y


def silu(v):
    return float(lib().orc_silu(float(v)))


def sigmoid(v):
    return float(lib().orc_sigmoid(float(v)))


def rms_norm(x, alpha, eps):
    x = _f32(x)
    alpha = _f32(alpha)
    y = np.empty_like(x)
    lib().orc_rms_norm(_p(x), x.size // x.shape[-1], x.shape[-1], _p(alpha), eps, _p(y))
    return y


def gate_logits(xs, wg):
    xs, wg = _f32(xs), _f32(wg)
    T, H = xs.shape
    E = wg.shape[0]
    out = np.empty((T, E), dtype=np.float32)
    lib().orc_gate_logits(_p(xs), T, H, _p(wg), E, _p(out))
    return out


def route(probs, k, norm_topk=True):
    probs = _f32(probs)
    T, E = probs.shape
    idx = np.zeros((T, k), dtype=np.int32)
    w = np.zeros((T, k), dtype=np.float32)
    offsets = np.zeros(E + 1, dtype=np.int32)
    perm = np.zeros(T * k, dtype=np.int32)
    perm_w = np.zeros(T * k, dtype=np.float32)
    rc = lib().orc_route(_p(probs), T, E, k, int(norm_topk), _p(idx), _p(w), _p(offsets), _p(perm), _p(perm_w))
    assert rc == 0
    return idx, w, offsets, perm, perm_w


def fill_normal(seed, n, mean=0.0, std=1.0, threads=8):
    out = np.empty(n, dtype=np.float32)
    lib().orc_fill_normal(seed, n, mean, std, _p(out), threads)
    return out


def fill_normal_quantized(seed, dtype, rows, k, std, threads=8):
    out = np.zeros(nbytes(dtype, rows * k), dtype=np.uint8)
    assert lib().orc_fill_normal_quantized(seed, dtype, rows, k, std, _p(out), threads) == 0
    return out


class Layer:
    """Block-level oracle: candle's MlpOrMoe::MoE forward on raw GGUF blocks."""

    def __init__(self, H, F, E, k, dtype, gate, w1, w3, w2, norm_topk=True, gate_bias=None,
                 Fs=0, sw1=None, sw3=None, sw2=None, shared_gate=None, rms_alpha=None, rms_eps=1e-5, dtype_down=None,
                 gate_dtype=None, gate_blocks=None):
        """gate_dtype / gate_blocks: the router tensor kept quantised, the `QMatMul::QTensor` arm that
        `QMatMul::from_arc` (candle-core/src/quantized/mod.rs:428-447) takes for every dtype but F32 / F16 / BF16: the
        logits are then `k_quants::matmul` (k_quants.rs:1873-1920) of the rows the block sees against those blocks."""
        self.H, self.F, self.E, self.k, self.dtype = H, F, E, k, dtype
        self.gate_dtype, self.gate_blocks, self.rms_eps = gate_dtype, gate_blocks, rms_eps
        if gate_dtype:
            assert np.asarray(gate_blocks).size == nbytes(gate_dtype, E * H)
            gate = np.zeros((E, H), dtype=np.float32) if gate is None else gate
        self.dtype_down = dtype if dtype_down is None else dtype_down
        self._keep = []

        def keep(a, dt):
            if a is None:
                return None
            a = np.ascontiguousarray(a, dtype=dt)
            self._keep.append(a)
            return a

        self.gate = keep(gate, np.float32)
        self.gate_bias = keep(gate_bias, np.float32)
        self.w1 = [keep(w, np.uint8) for w in w1]
        self.w3 = [keep(w, np.uint8) for w in w3]
        self.w2 = [keep(w, np.uint8) for w in w2]
        for w in self.w1 + self.w3:
            assert w.size == nbytes(dtype, H * F)
        for w in self.w2:
            assert w.size == nbytes(self.dtype_down, H * F)
        self.sw = [keep(w, np.uint8) for w in (sw1, sw3, sw2)]
        self.shared_gate = keep(shared_gate, np.float32)
        self.rms_alpha = keep(rms_alpha, np.float32)
        arr = lambda ws: (C.c_void_p * E)(*[w.ctypes.data for w in ws])
        self._a1, self._a3, self._a2 = arr(self.w1), arr(self.w3), arr(self.w2)
        ptr = lambda a: None if a is None else a.ctypes.data
        self.c = _Layer(H, F, E, k, dtype, int(norm_topk), ptr(self.gate), ptr(self.gate_bias),
                        C.cast(self._a1, C.POINTER(C.c_void_p)), C.cast(self._a3, C.POINTER(C.c_void_p)),
                        C.cast(self._a2, C.POINTER(C.c_void_p)), Fs, ptr(self.sw[0]), ptr(self.sw[1]),
                        ptr(self.sw[2]), ptr(self.shared_gate), ptr(self.rms_alpha), rms_eps,
                        0 if self.dtype_down == dtype else self.dtype_down)

    def router_logits(self, xs, simd=False):
        """Logits of the quantised router (`self.gate_blocks`) on the rows the block sees: after the pre-norm when the
        layer carries one (quantized_llama.rs:886-890), plus the bias."""
        seen = _f32(xs) if self.rms_alpha is None else rms_norm(xs, self.rms_alpha, self.rms_eps)
        lo = matmul(self.gate_dtype, seen, self.gate_blocks, self.E, simd=simd)
        return lo if self.gate_bias is None else (lo + self.gate_bias[None, :]).astype(np.float32)

    def forward(self, xs, logits=None, simd=False, threads=1, return_logits=False):
        xs = _f32(xs)
        T = xs.shape[0]
        if logits is None and self.gate_dtype:
            logits = self.router_logits(xs, simd=simd)
        ys = np.empty((T, self.H), dtype=np.float32)
        lo = np.empty((T, self.E), dtype=np.float32)
        li = None if logits is None else _f32(logits)
        rc = lib().orc_moe_forward(C.byref(self.c), _p(xs), T, None if li is None else _p(li), _p(lo),
                                   _p(ys), int(simd), threads)
        assert rc == 0
        return (ys, lo) if return_logits else ys
