"""CPU-side checks of the shipped library: it loads, exports everything the header declares,
refuses to compute without a GPU (no fallback), and its exp restatement equals the platform expf."""
import ctypes
import os
import re

import numpy as np
import pytest

import candle_amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    src = open(os.path.join(ROOT, "include", "candle_amd_moe.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    lib = candle_amd.load_library()
    names = declared_functions()
    assert {"moe_layer_create", "moe_layer_forward", "moe_layer_forward_device", "moe_route", "moe_dequantize",
            "moe_quantize_act", "moe_last_error", "moe_layer_destroy"} <= set(names)
    for n in names:
        assert getattr(lib, n) is not None, n


def test_build_id_names_the_sources_on_disk():
    # the library in the tree was compiled from the sources in the tree (a stale library would carry another id)
    from candle_amd import build
    assert re.fullmatch(r"[0-9a-f]{16}", candle_amd.build_id())
    assert candle_amd.build_id() == build.source_id()


def test_header_is_plain_c(tmp_path):
    # the boundary is a C ABI: the header has to compile as C99 (no C++ in the signatures), and a C caller has to link
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if not gcc:
        pytest.skip("no gcc")
    src = tmp_path / "caller.c"
    src.write_text('#include "candle_amd_moe.h"\n'
                   'int main(void) { moe_desc d; (void)d; return moe_static_scratch_bytes() > 0 && moe_last_error() ? 0 : 1; }\n')
    lib = candle_amd.lib_path()
    exe = tmp_path / "caller"
    subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                    "-L", os.path.dirname(lib), "-lcandle_amd_moe", "-Wl,-rpath," + os.path.dirname(lib)], check=True)
    assert subprocess.run([str(exe)]).returncode == 0


def test_debug_expf_equals_platform_expf():
    libm = ctypes.CDLL("libm.so.6")
    libm.expf.restype = ctypes.c_float
    libm.expf.argtypes = [ctypes.c_float]
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.uniform(-104, 89, 20000), rng.uniform(-20, 0, 40000), rng.normal(0, 1e-3, 2000),
                         [0.0, -0.0, 88.72283, 88.7229, -103.97, -103.98, -87.3, -1e-30, np.inf, -np.inf]]).astype(np.float32)
    for x in xs:
        a, b = candle_amd.debug_expf(float(x)), libm.expf(float(x))
        assert a == b, (x, a, b)
    assert np.isnan(candle_amd.debug_expf(float("nan")))


def test_no_gpu_means_error_not_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(candle_amd.MoeError, match="no CPU fallback"):
        candle_amd.dequantize(candle_amd.GGML_Q4_0, np.zeros(18, np.uint8), 32)
    with pytest.raises(candle_amd.MoeError):
        candle_amd.route(np.zeros((2, 8), np.float32), 2)
