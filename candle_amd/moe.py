"""ctypes binding of libcandle_amd_moe.so.

`SparseMoeBlock.forward(xs)` takes the same `[b, seq, hidden]` (or `[tokens, hidden]`) f32
activations as `MlpOrMoe::forward` (candle-transformers/src/models/quantized_llama.rs:143-211)
and returns the same shape.  numpy arrays go through the host entry point (as candle's
`CustomOp1::cpu_fwd` would); torch CUDA tensors go through the device entry point on torch's
current stream.
"""
import ctypes as C
import os

import numpy as np

GGML_Q4_0, GGML_Q4_1, GGML_Q5_0, GGML_Q5_1, GGML_Q8_0, GGML_Q8_1 = 2, 3, 6, 7, 8, 9
GGML_Q2K, GGML_Q3K, GGML_Q4K, GGML_Q5K, GGML_Q6K, GGML_Q8K = 10, 11, 12, 13, 14, 15
_BLOCK = {GGML_Q4_0: (32, 18), GGML_Q4_1: (32, 20), GGML_Q5_0: (32, 22), GGML_Q5_1: (32, 24), GGML_Q8_0: (32, 34), GGML_Q8_1: (32, 36),
          GGML_Q2K: (256, 84), GGML_Q3K: (256, 110), GGML_Q4K: (256, 144), GGML_Q5K: (256, 176), GGML_Q6K: (256, 210),
          GGML_Q8K: (256, 292)}

_HERE = os.path.dirname(os.path.abspath(__file__))
# CANDLE_AMD_MOE_LIB points at another build of the library (a tuning experiment built beside the product's)
_LIB_PATH = os.environ.get("CANDLE_AMD_MOE_LIB") or os.path.join(_HERE, "lib", "libcandle_amd_moe.so")
_lib = None


class MoeError(RuntimeError):
    """Mirrors candle::Error::Msg: carries the library's message."""


class _Desc(C.Structure):
    _fields_ = [
        ("hidden", C.c_int64), ("ffn", C.c_int64), ("n_experts", C.c_int64), ("top_k", C.c_int64),
        ("ggml_dtype", C.c_int32), ("norm_topk", C.c_int32),
        ("gate", C.c_void_p), ("gate_bias", C.c_void_p),
        ("w1", C.POINTER(C.c_void_p)), ("w3", C.POINTER(C.c_void_p)), ("w2", C.POINTER(C.c_void_p)),
        ("shared_ffn", C.c_int64), ("shared_w1", C.c_void_p), ("shared_w3", C.c_void_p), ("shared_w2", C.c_void_p),
        ("shared_gate", C.c_void_p), ("rms_alpha", C.c_void_p), ("rms_eps", C.c_float),
        ("ggml_dtype_down", C.c_int32),
        ("gate_dtype", C.c_int32), ("gate_blocks", C.c_void_p),
    ]


def lib_path():
    return _LIB_PATH


def load_library():
    """Loads the built library; raises if it has not been built (no fallback path exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise MoeError("%s is missing: build it with `python -m candle_amd.build` "
                       "(there is no CPU fallback)" % _LIB_PATH)
    # A process must hold ONE HIP runtime.  PyTorch ships its own libamdhip64; if this library
    # pulled in the system copy first, torch would later fail with "No HIP GPUs are available".
    # Importing torch first makes the loader resolve our dependency to the copy torch uses.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(_LIB_PATH)
    vp, i64, i32 = C.c_void_p, C.c_int64, C.c_int32
    L.moe_layer_create.argtypes = [C.POINTER(_Desc), C.POINTER(vp)]
    L.moe_layer_destroy.argtypes = [vp]
    L.moe_layer_destroy.restype = None
    L.moe_layer_forward.argtypes = [vp, vp, i64, vp]
    L.moe_layer_forward_device.argtypes = [vp, vp, i64, vp, vp]
    L.moe_layer_forward_device_noalloc.argtypes = [vp, vp, i64, vp, vp]
    L.moe_static_scratch_bytes.restype = i64
    L.moe_stack_forward_device.argtypes = [C.POINTER(vp), i64, vp, i64, vp, vp]
    L.moe_layer_forward_timed.argtypes = [vp, vp, i64, vp, vp, vp]
    L.moe_rms_norm.argtypes = [vp, vp, C.c_float, i64, i64, vp]
    L.moe_add_rms_norm_device.argtypes = [vp, vp, vp, C.c_float, i64, i64, vp, vp, vp]
    L.moe_debug_set_switch.argtypes = [C.c_char_p, i64]
    L.moe_layer_last_logits.argtypes = [vp, vp, i64]
    L.moe_layer_last_routing.argtypes = [vp, i64, vp, vp, vp, vp, vp]
    L.moe_layer_dequantize_weight.argtypes = [vp, i64, C.c_int, vp, i64]
    L.moe_route.argtypes = [vp, i64, i64, i64, i32, vp, vp, vp, vp, vp]
    L.moe_dequantize.argtypes = [i32, vp, i64, vp]
    L.moe_quantize_act.argtypes = [i32, vp, i64, i64, vp]
    L.moe_qmatmul.argtypes = [i32, vp, i64, i64, vp, i64, vp]
    L.moe_qlinear_create.argtypes = [i32, vp, i64, i64, C.POINTER(vp)]
    L.moe_qlinear_destroy.argtypes = [vp]
    L.moe_qlinear_destroy.restype = None
    L.moe_qlinear_forward.argtypes = [vp, vp, i64, vp]
    L.moe_qlinear_forward_device.argtypes = [vp, vp, i64, vp, vp]
    L.moe_qlinear_dequantize.argtypes = [vp, vp, i64]
    L.moe_qlinear_shape.argtypes = [vp, C.POINTER(i64), C.POINTER(i64), C.POINTER(i32)]
    L.moe_qlinear_create_from_gguf.argtypes = [vp, C.c_char_p, C.POINTER(vp)]
    L.moe_quantize_weights.argtypes = [i32, vp, i64, vp]
    L.moe_quantize_weights_device.argtypes = [i32, vp, i64, vp, vp]
    L.moe_gguf_open.argtypes = [C.c_char_p, C.POINTER(vp)]
    L.moe_gguf_close.argtypes = [vp]
    L.moe_gguf_close.restype = None
    L.moe_gguf_version.argtypes = [vp]
    L.moe_gguf_tensor_count.argtypes = [vp]
    L.moe_gguf_tensor_count.restype = i64
    L.moe_gguf_tensor_data_offset.argtypes = [vp]
    L.moe_gguf_tensor_data_offset.restype = C.c_uint64
    L.moe_gguf_tensor_name.argtypes = [vp, i64]
    L.moe_gguf_tensor_name.restype = C.c_char_p
    L.moe_gguf_metadata_type.argtypes = [vp, C.c_char_p, C.POINTER(C.c_int)]
    L.moe_gguf_metadata_u64.argtypes = [vp, C.c_char_p, C.POINTER(C.c_uint64)]
    L.moe_gguf_metadata_i64.argtypes = [vp, C.c_char_p, C.POINTER(C.c_int64)]
    L.moe_gguf_metadata_f64.argtypes = [vp, C.c_char_p, C.POINTER(C.c_double)]
    L.moe_gguf_metadata_str.argtypes = [vp, C.c_char_p, C.c_char_p, C.c_uint64]
    L.moe_gguf_metadata_array_len.argtypes = [vp, C.c_char_p, C.POINTER(C.c_uint64), C.POINTER(C.c_int)]
    L.moe_gguf_tensor.argtypes = [vp, C.c_char_p, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(i64), C.POINTER(vp), C.POINTER(C.c_uint64)]
    L.moe_layer_create_from_gguf.argtypes = [vp, C.c_int, C.c_int, C.POINTER(vp)]
    L.moe_last_error.restype = C.c_char_p
    L.moe_device_arch.restype = C.c_char_p
    L.moe_build_id.restype = C.c_char_p
    L.moe_debug_expf.restype = C.c_float
    L.moe_debug_expf.argtypes = [C.c_float]
    _lib = L
    return L


def _check(rc):
    if rc != 0:
        raise MoeError(load_library().moe_last_error().decode())


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    a = np.asarray(a)
    if a.dtype != np.float32:
        raise MoeError("expected f32 activations, got %s" % a.dtype)  # the reference bails on other dtypes
    return np.ascontiguousarray(a)


def _blocks(a, dtype, n_elems, what):
    a = np.ascontiguousarray(np.asarray(a).view(np.uint8).reshape(-1))
    be, bb = _BLOCK[dtype]
    if n_elems % be or a.size != n_elems // be * bb:
        raise MoeError("%s: expected %d bytes of dtype %d blocks, got %d" % (what, n_elems // be * bb, dtype, a.size))
    return a


def device_arch():
    r = load_library().moe_device_arch()
    if r is None:
        raise MoeError(load_library().moe_last_error().decode())
    return r.decode()


def build_id():
    """The id of the sources the loaded library was compiled from (moe_build_id)."""
    return load_library().moe_build_id().decode()


def debug_expf(x):
    return float(load_library().moe_debug_expf(float(x)))


def set_switch(name, value):
    """Test aid: sets a process-wide tuning switch of the library (see moe_debug_set_switch)."""
    _check(load_library().moe_debug_set_switch(name.encode(), int(value)))


def static_scratch_bytes():
    return int(load_library().moe_static_scratch_bytes())


def rms_norm(x, alpha, eps, residual=None):
    """`RmsNorm::forward` (candle-transformers/src/quantized_nn.rs:100-126) on rows of f32.  numpy in -> numpy out
    (host entry); torch CUDA tensors go through the device entry on torch's current stream.  With `residual`
    (device tensors only) returns (x + residual, rms_norm(x + residual))."""
    L = load_library()
    if isinstance(x, np.ndarray):
        if residual is not None:
            raise MoeError("the host entry takes no residual")
        x, alpha = _f32(x), _f32(alpha)
        hidden = x.shape[-1]
        if alpha.size != hidden:
            raise MoeError("alpha must have %d elements" % hidden)
        y = np.empty_like(x)
        _check(L.moe_rms_norm(_p(x), _p(alpha), float(eps), x.size // hidden, hidden, _p(y)))
        return y
    import torch
    ok = lambda t: isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
    if not ok(x) or not ok(alpha) or (residual is not None and not ok(residual)):
        raise MoeError("rms_norm takes numpy arrays or contiguous f32 torch CUDA tensors")
    hidden = x.shape[-1]
    if alpha.numel() != hidden or (residual is not None and residual.shape != x.shape):
        raise MoeError("shape mismatch")
    y = torch.empty_like(x)
    total = torch.empty_like(x) if residual is not None else None
    stream = torch.cuda.current_stream(x.device).cuda_stream
    _check(L.moe_add_rms_norm_device(x.data_ptr(), None if residual is None else residual.data_ptr(), alpha.data_ptr(), float(eps),
                                     x.numel() // hidden, hidden, None if total is None else total.data_ptr(), y.data_ptr(), stream))
    return y if residual is None else (total, y)


def dequantize(dtype, blocks, n_elems):
    """GgmlType::to_float on the GPU (parity hook)."""
    blocks = _blocks(blocks, dtype, n_elems, "dequantize")
    out = np.empty(n_elems, dtype=np.float32)
    _check(load_library().moe_dequantize(dtype, _p(blocks), n_elems, _p(out)))
    return out


def quantize_act(vecdot_dtype, x):
    """The activation quantiser of k_quants::matmul on the GPU; returns raw BlockQ8_0 / BlockQ8K bytes."""
    x = _f32(x)
    rows, k = (1, x.size) if x.ndim == 1 else (x.shape[0], x.shape[1])
    be, bb = _BLOCK[vecdot_dtype]
    out = np.zeros(rows * k // be * bb, dtype=np.uint8)
    _check(load_library().moe_quantize_act(vecdot_dtype, _p(x), rows, k, _p(out)))
    return out


def route(logits, top_k, norm_topk=True):
    """softmax + top-k + per-expert lists on the GPU given router logits (parity hook)."""
    logits = _f32(logits)
    T, E = logits.shape
    idx = np.zeros((T, top_k), dtype=np.int32)
    w = np.zeros((T, top_k), dtype=np.float32)
    offsets = np.zeros(E + 1, dtype=np.int32)
    perm = np.zeros(T * top_k, dtype=np.int32)
    perm_w = np.zeros(T * top_k, dtype=np.float32)
    _check(load_library().moe_route(_p(logits), T, E, top_k, int(norm_topk), _p(idx), _p(w), _p(offsets), _p(perm), _p(perm_w)))
    return idx, w, offsets, perm, perm_w


def qmatmul(dtype, w_blocks, n, k, x):
    """QMatMul::forward of one quantized [n, k] matrix on the GPU: x [m, k] -> [m, n]."""
    x = _f32(x)
    m = x.shape[0]
    w_blocks = _blocks(w_blocks, dtype, n * k, "qmatmul")
    y = np.empty((m, n), dtype=np.float32)
    _check(load_library().moe_qmatmul(dtype, _p(w_blocks), n, k, _p(x), m, _p(y)))
    return y


def quantize_weights(dtype, x):
    """QTensor::quantize on the GPU.  numpy f32 in -> numpy uint8 blocks out; a torch CUDA f32
    tensor in -> a torch CUDA uint8 tensor out (enqueued on torch's current stream)."""
    L = load_library()
    be, bb = _BLOCK[dtype]
    if isinstance(x, np.ndarray):
        x = _f32(x)
        if x.size % be or (x.ndim > 1 and x.shape[-1] % be):
            raise MoeError("last dimension must be a multiple of the block size %d" % be)
        out = np.zeros(x.size // be * bb, dtype=np.uint8)
        _check(L.moe_quantize_weights(dtype, _p(x), x.size, _p(out)))
        return out
    import torch
    if not (isinstance(x, torch.Tensor) and x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()):
        raise MoeError("quantize_weights takes a numpy f32 array or a contiguous f32 torch CUDA tensor")
    if x.shape[-1] % be:
        raise MoeError("last dimension must be a multiple of the block size %d" % be)
    out = torch.empty(x.numel() // be * bb, dtype=torch.uint8, device=x.device)
    _check(L.moe_quantize_weights_device(dtype, x.data_ptr(), x.numel(), out.data_ptr(),
                                         torch.cuda.current_stream(x.device).cuda_stream))
    return out


class GgufFile:
    """A memory-mapped GGUF file (`gguf_file::Content`): metadata, tensor table, tensor bytes."""

    def __init__(self, path):
        self._h = None
        h = C.c_void_p()
        _check(load_library().moe_gguf_open(os.fsencode(path), C.byref(h)))
        self._h = h

    def close(self):
        if getattr(self, "_h", None) is not None:
            load_library().moe_gguf_close(self._h)
            self._h = None

    __del__ = close

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    @property
    def version(self):
        return load_library().moe_gguf_version(self._h)

    @property
    def tensor_data_offset(self):
        return load_library().moe_gguf_tensor_data_offset(self._h)

    def tensor_names(self):
        L = load_library()
        return [L.moe_gguf_tensor_name(self._h, i).decode() for i in range(L.moe_gguf_tensor_count(self._h))]

    def metadata(self, key):
        """The value of a metadata key as int / float / bool / str, or ("array", length, element type id)."""
        L = load_library()
        k = key.encode()
        vt = C.c_int()
        _check(L.moe_gguf_metadata_type(self._h, k, C.byref(vt)))
        if vt.value in (0, 2, 4, 7, 10):
            v = C.c_uint64()
            _check(L.moe_gguf_metadata_u64(self._h, k, C.byref(v)))
            return bool(v.value) if vt.value == 7 else v.value
        if vt.value in (1, 3, 5, 11):
            v = C.c_int64()
            _check(L.moe_gguf_metadata_i64(self._h, k, C.byref(v)))
            return v.value
        if vt.value in (6, 12):
            v = C.c_double()
            _check(L.moe_gguf_metadata_f64(self._h, k, C.byref(v)))
            return v.value
        if vt.value == 8:
            buf = C.create_string_buffer(1 << 16)
            _check(L.moe_gguf_metadata_str(self._h, k, buf, len(buf)))
            return buf.value.decode(errors="replace")
        n, et = C.c_uint64(), C.c_int()
        _check(L.moe_gguf_metadata_array_len(self._h, k, C.byref(n), C.byref(et)))
        return ("array", n.value, et.value)

    def metadata_u32_or_zero(self, key):
        """`md_get(key).and_then(|v| v.to_u32()).unwrap_or(0)`: the value of a U32 key, 0 for a missing key and for
        one of any other type (`Value::to_u32`, gguf_file.rs:249-254, takes the U32 variant only)."""
        vt = C.c_int()
        if load_library().moe_gguf_metadata_type(self._h, key.encode(), C.byref(vt)) or vt.value != 4:
            return 0
        return int(self.metadata(key))

    def tensor(self, name):
        """(ggml dtype id, shape, bytes as a numpy uint8 view of the mapping)."""
        L = load_library()
        dt, nd, dims, data, nbytes = C.c_int(), C.c_int(), (C.c_int64 * 8)(), C.c_void_p(), C.c_uint64()
        _check(L.moe_gguf_tensor(self._h, name.encode(), C.byref(dt), C.byref(nd), dims, C.byref(data), C.byref(nbytes)))
        raw = np.ctypeslib.as_array(C.cast(data, C.POINTER(C.c_uint8)), shape=(nbytes.value,)) if nbytes.value else np.zeros(0, np.uint8)
        return dt.value, tuple(dims[i] for i in range(nd.value)), raw


class SparseMoeBlock:
    """The MoE arm of `MlpOrMoe` with quantized experts resident on the GPU.

    gate: f32 [E, H]; w1/w3: E raw block arrays of [F, H]; w2: E raw block arrays of [H, F]
    (the bytes of candle's `QTensor::data()`).
    """

    def __init__(self, hidden, ffn, n_experts, top_k, ggml_dtype, gate, w1, w3, w2, norm_topk=True,
                 gate_bias=None, shared_ffn=0, shared_w1=None, shared_w3=None, shared_w2=None,
                 shared_gate=None, rms_alpha=None, rms_eps=1e-5, ggml_dtype_down=None, gate_dtype=None, gate_blocks=None):
        """gate_dtype / gate_blocks: a router tensor kept quantised, as the reference keeps every `ffn_gate_inp` that is
        not F32 / F16 / BF16 (`QMatMul::from_arc`, quantized/mod.rs:428-447): the raw blocks of the [E, H] tensor; `gate`
        is then ignored and may be None."""
        L = load_library()
        dtype_down = ggml_dtype if ggml_dtype_down is None else ggml_dtype_down
        for dt in (ggml_dtype, dtype_down):
            if dt not in _BLOCK or dt in (GGML_Q8K, GGML_Q8_1):
                raise MoeError("unsupported ggml_dtype %r" % (dt,))
        self.dtype_down = dtype_down
        if len(w1) != n_experts or len(w2) != n_experts or len(w3) != n_experts:
            raise MoeError("need one w1/w2/w3 per expert")
        self.hidden, self.ffn, self.n_experts, self.top_k, self.dtype = hidden, ffn, n_experts, top_k, ggml_dtype
        self.shared_ffn = shared_ffn
        if gate_dtype:
            if gate_dtype not in _BLOCK or gate_dtype in (GGML_Q8K, GGML_Q8_1):
                raise MoeError("unsupported gate_dtype %r" % (gate_dtype,))
            gate_q = _blocks(gate_blocks, gate_dtype, n_experts * hidden, "gate_blocks")
            gate = np.zeros((n_experts, hidden), dtype=np.float32)   # not read by the library
            keep = [gate, gate_q]
        else:
            gate_q = None
            gate = _f32(gate).reshape(n_experts, hidden)
            keep = [gate]
        mats = {}
        for name, ws in (("w1", w1), ("w3", w3), ("w2", w2)):
            arrs = [_blocks(w, dtype_down if name == "w2" else ggml_dtype, hidden * ffn, name) for w in ws]
            keep += arrs
            mats[name] = (C.c_void_p * n_experts)(*[a.ctypes.data for a in arrs])
        opt = {}
        for name, a, n in (("gate_bias", gate_bias, n_experts), ("shared_gate", shared_gate, hidden), ("rms_alpha", rms_alpha, hidden)):
            if a is not None:
                a = _f32(a).reshape(n)
                keep.append(a)
            opt[name] = a
        sh = {}
        for name, a in (("shared_w1", shared_w1), ("shared_w3", shared_w3), ("shared_w2", shared_w2)):
            if shared_ffn:
                a = _blocks(a, dtype_down if name == "shared_w2" else ggml_dtype, hidden * shared_ffn, name)
                keep.append(a)
            else:
                a = None
            sh[name] = a
        ptr = lambda a: None if a is None else a.ctypes.data
        desc = _Desc(hidden, ffn, n_experts, top_k, ggml_dtype, int(norm_topk), ptr(gate), ptr(opt["gate_bias"]),
                     C.cast(mats["w1"], C.POINTER(C.c_void_p)), C.cast(mats["w3"], C.POINTER(C.c_void_p)),
                     C.cast(mats["w2"], C.POINTER(C.c_void_p)), shared_ffn, ptr(sh["shared_w1"]), ptr(sh["shared_w3"]),
                     ptr(sh["shared_w2"]), ptr(opt["shared_gate"]), ptr(opt["rms_alpha"]), float(rms_eps),
                     0 if dtype_down == ggml_dtype else dtype_down, int(gate_dtype or 0), ptr(gate_q))
        handle = C.c_void_p()
        self._h = None
        _check(L.moe_layer_create(C.byref(desc), C.byref(handle)))
        self._h = handle
        del keep  # host copies are only borrowed during create

    @classmethod
    def from_gguf(cls, gguf, layer_index, norm_topk=True):
        """The MoE block of layer `layer_index` of a GGUF file (a path or an open GgufFile), as
        `ModelWeights::from_gguf` builds it (quantized_llama.rs:506-512, 553-578)."""
        own = not isinstance(gguf, GgufFile)
        g = GgufFile(gguf) if own else gguf
        try:
            h = C.c_void_p()
            _check(load_library().moe_layer_create_from_gguf(g._h, int(layer_index), int(norm_topk), C.byref(h)))
            prefix = "blk.%d" % layer_index
            dt, (f, hdim), _ = g.tensor(prefix + ".ffn_gate.0.weight")
            self = cls.__new__(cls)
            self._h = h
            self.hidden, self.ffn, self.dtype = hdim, f, dt
            self.dtype_down = g.tensor(prefix + ".ffn_down.0.weight")[0]
            # the reference's default for a missing key or one that is not a U32 is 0 (quantized_llama.rs:507-512)
            self.n_experts = g.metadata_u32_or_zero("llama.expert_count")
            self.top_k = g.metadata_u32_or_zero("llama.expert_used_count")
            self.shared_ffn = 0
            return self
        finally:
            if own:
                g.close()

    def close(self):
        if getattr(self, "_h", None) is not None:
            load_library().moe_layer_destroy(self._h)
            self._h = None

    __del__ = close

    def forward(self, xs, out=None, noalloc=False):
        """noalloc (device tensors only): the entry point that allocates nothing (workspace in the library's static
        device array; fails for batches beyond it)."""
        L = load_library()
        if self._h is None:
            raise MoeError("layer is closed")
        if isinstance(xs, np.ndarray):
            if noalloc:
                raise MoeError("noalloc applies to device tensors")
            x = _f32(xs)
            if x.ndim not in (2, 3) or x.shape[-1] != self.hidden:
                raise MoeError("expected [b, seq, %d] or [tokens, %d], got %s" % (self.hidden, self.hidden, x.shape))
            T = x.size // self.hidden
            y = np.empty_like(x)
            _check(L.moe_layer_forward(self._h, _p(x), T, _p(y)))
            return y
        import torch  # device tensors: plumbing only
        if not (isinstance(xs, torch.Tensor) and xs.is_cuda):
            raise MoeError("forward takes a numpy array or a torch CUDA tensor")
        if xs.dtype != torch.float32 or not xs.is_contiguous():
            raise MoeError("input has to be contiguous f32")
        if xs.dim() not in (2, 3) or xs.shape[-1] != self.hidden:
            raise MoeError("expected [b, seq, %d] or [tokens, %d], got %s" % (self.hidden, self.hidden, tuple(xs.shape)))
        T = xs.numel() // self.hidden
        y = torch.empty_like(xs) if out is None else out
        stream = torch.cuda.current_stream(xs.device).cuda_stream
        entry = L.moe_layer_forward_device_noalloc if noalloc else L.moe_layer_forward_device
        _check(entry(self._h, xs.data_ptr(), T, y.data_ptr(), stream))
        return y

    __call__ = forward

    STAGES = ("front", "dispatch", "up", "requant", "down", "shared", "combine")

    def forward_timed(self, xs, out):
        """One forward on torch CUDA tensors with HIP events between the launches (on torch's
        current stream); returns {stage: milliseconds}.  Synchronises."""
        import torch
        T = xs.numel() // self.hidden
        ms = (C.c_float * len(self.STAGES))()
        stream = torch.cuda.current_stream(xs.device).cuda_stream
        _check(load_library().moe_layer_forward_timed(self._h, xs.data_ptr(), T, out.data_ptr(), stream, ms))
        return dict(zip(self.STAGES, [float(v) for v in ms]))

    def last_logits(self, n_tokens):
        out = np.empty((n_tokens, self.n_experts), dtype=np.float32)
        _check(load_library().moe_layer_last_logits(self._h, _p(out), n_tokens))
        return out

    def last_routing(self, n_tokens):
        k, E = self.top_k, self.n_experts
        idx = np.zeros((n_tokens, k), dtype=np.int32)
        w = np.zeros((n_tokens, k), dtype=np.float32)
        offsets = np.zeros(E + 1, dtype=np.int32)
        perm = np.zeros(n_tokens * k, dtype=np.int32)
        perm_w = np.zeros(n_tokens * k, dtype=np.float32)
        _check(load_library().moe_layer_last_routing(self._h, n_tokens, _p(idx), _p(w), _p(offsets), _p(perm), _p(perm_w)))
        return idx, w, offsets, perm, perm_w

    def dequantize_weight(self, expert, which):
        """to_float of matrix `which` (1, 2, 3) of `expert` (E = shared expert) read back from the device layout."""
        F = self.shared_ffn if expert == self.n_experts else self.ffn
        out = np.empty(self.hidden * F, dtype=np.float32)
        _check(load_library().moe_layer_dequantize_weight(self._h, expert, which, _p(out), out.size))
        return out.reshape((self.hidden, F) if which == 2 else (F, self.hidden))


MlpOrMoe = SparseMoeBlock  # the reference's name for the enum that holds the MoE arm


def stack_forward(layers, xs, out=None):
    """`layers[-1](... layers[1](layers[0](xs)))` for a list of SparseMoeBlocks on a contiguous f32 torch CUDA tensor
    (torch's current stream): the same bits as calling the layers one by one, with each layer's combine pass folded
    into the next layer's front kernel where the batch is small (moe_stack_forward_device)."""
    import torch
    if not layers:
        raise MoeError("stack_forward needs at least one layer")
    if not (isinstance(xs, torch.Tensor) and xs.is_cuda and xs.dtype == torch.float32 and xs.is_contiguous()):
        raise MoeError("stack_forward takes a contiguous f32 torch CUDA tensor")
    hidden = layers[0].hidden
    if xs.dim() not in (2, 3) or xs.shape[-1] != hidden:
        raise MoeError("expected [b, seq, %d] or [tokens, %d], got %s" % (hidden, hidden, tuple(xs.shape)))
    for layer in layers:
        if layer._h is None:
            raise MoeError("layer is closed")
    y = torch.empty_like(xs) if out is None else out
    handles = (C.c_void_p * len(layers))(*[layer._h for layer in layers])
    stream = torch.cuda.current_stream(xs.device).cuda_stream
    _check(load_library().moe_stack_forward_device(handles, len(layers), xs.data_ptr(), xs.numel() // hidden, y.data_ptr(), stream))
    return y


class QMatMul:
    """The `QMatMul::QTensor` arm (candle-core/src/quantized/mod.rs:428-447, 533-537): one quantized
    [n, k] matrix resident on the GPU, applied as xs . W^T (the attention and output projections
    of quantized_llama.rs:590-593, 608)."""

    def __init__(self, ggml_dtype, w_blocks, n, k):
        if ggml_dtype not in _BLOCK or ggml_dtype in (GGML_Q8K, GGML_Q8_1):
            raise MoeError("unsupported ggml_dtype %r" % (ggml_dtype,))
        w_blocks = _blocks(w_blocks, ggml_dtype, n * k, "QMatMul")
        h = C.c_void_p()
        self._h = None
        _check(load_library().moe_qlinear_create(ggml_dtype, _p(w_blocks), n, k, C.byref(h)))
        self._h, self.n, self.k, self.dtype = h, n, k, ggml_dtype

    from_qtensor = classmethod(lambda cls, ggml_dtype, w_blocks, n, k: cls(ggml_dtype, w_blocks, n, k))

    @classmethod
    def from_gguf(cls, gguf, tensor_name):
        """`QMatMul::from_qtensor(ct.tensor(reader, name, device)?)` (quantized_llama.rs:533-547)."""
        own = not isinstance(gguf, GgufFile)
        g = GgufFile(gguf) if own else gguf
        try:
            L = load_library()
            h = C.c_void_p()
            _check(L.moe_qlinear_create_from_gguf(g._h, tensor_name.encode(), C.byref(h)))
            n, k, dt = C.c_int64(), C.c_int64(), C.c_int32()
            self = cls.__new__(cls)
            self._h = h
            _check(L.moe_qlinear_shape(h, C.byref(n), C.byref(k), C.byref(dt)))
            self.n, self.k, self.dtype = n.value, k.value, dt.value
            return self
        finally:
            if own:
                g.close()

    def close(self):
        if getattr(self, "_h", None) is not None:
            load_library().moe_qlinear_destroy(self._h)
            self._h = None

    __del__ = close

    def forward(self, xs, out=None):
        """xs [..., k] f32 (numpy, or a contiguous torch CUDA tensor on torch's current stream) -> [..., n]."""
        L = load_library()
        if self._h is None:
            raise MoeError("QMatMul is closed")
        if isinstance(xs, np.ndarray):
            x = _f32(xs)
            if x.ndim < 1 or x.shape[-1] != self.k:
                raise MoeError("expected [..., %d], got %s" % (self.k, x.shape))
            m = x.size // self.k
            y = np.empty(x.shape[:-1] + (self.n,), dtype=np.float32)
            _check(L.moe_qlinear_forward(self._h, _p(x), m, _p(y)))
            return y
        import torch  # device tensors: plumbing only
        if not (isinstance(xs, torch.Tensor) and xs.is_cuda):
            raise MoeError("forward takes a numpy array or a torch CUDA tensor")
        if xs.dtype != torch.float32 or not xs.is_contiguous():
            raise MoeError("input has to be contiguous f32")
        if xs.dim() < 1 or xs.shape[-1] != self.k:
            raise MoeError("expected [..., %d], got %s" % (self.k, tuple(xs.shape)))
        m = xs.numel() // self.k
        y = torch.empty(tuple(xs.shape[:-1]) + (self.n,), dtype=torch.float32, device=xs.device) if out is None else out
        if y.numel() != m * self.n or y.dtype != torch.float32 or not y.is_contiguous() or not y.is_cuda:
            raise MoeError("out has to be a contiguous f32 CUDA tensor of %d elements" % (m * self.n))
        stream = torch.cuda.current_stream(xs.device).cuda_stream
        _check(L.moe_qlinear_forward_device(self._h, xs.data_ptr(), m, y.data_ptr(), stream))
        return y

    __call__ = forward

    def dequantize(self):
        """`QMatMul::dequantize` of the resident copy: f32 [n, k]."""
        out = np.empty((self.n, self.k), dtype=np.float32)
        _check(load_library().moe_qlinear_dequantize(self._h, _p(out), out.size))
        return out
