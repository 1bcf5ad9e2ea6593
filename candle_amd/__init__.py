"""MI355X (gfx950) implementation of candle's quantized sparse-MoE block.

The product is the C-ABI shared library ``candle_amd/lib/libcandle_amd_moe.so`` (HIP kernels,
declared in ``include/candle_amd_moe.h``).  This package is a thin ctypes front end over it whose
classes mirror the names of the reference (``MlpOrMoe``/``SparseMoeBlock`` with ``forward``).
There is no CPU fallback: every call fails if the library or a gfx950 device is missing.
"""
from .moe import (  # noqa: F401
    GGML_Q4_0, GGML_Q4_1, GGML_Q5_0, GGML_Q5_1, GGML_Q8_0, GGML_Q8_1, GGML_Q2K, GGML_Q3K, GGML_Q4K, GGML_Q5K, GGML_Q6K, GGML_Q8K, MoeError, SparseMoeBlock, MlpOrMoe, QMatMul, GgufFile,
    dequantize, quantize_act, quantize_weights, route, qmatmul, device_arch, debug_expf, lib_path, load_library,
    set_switch, static_scratch_bytes, rms_norm, stack_forward, build_id,
)
