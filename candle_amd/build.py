"""Builds libcandle_amd_moe.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
import concurrent.futures
import hashlib
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(OUT_DIR, "libcandle_amd_moe.so")
SOURCES = ["api.hip", "kernels_front.hip", "kernels_util.hip", "kernels_q4k.hip", "kernels_q32.hip", "kernels_wquant.hip", "kernels_q4k_gemm.hip", "gguf.cpp"]

# -ffp-contract=off: candle's Rust never fuses a*b+c, and `to_float` / combine must round the
# product first to stay bit-exact.  Packed-FP32 instructions are switched off for the whole build.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def source_id(extra_flags=()):
    """Sixteen hex digits of the SHA-256 over the library's source files (names and contents, in name order) and any
    extra compiler flags: what moe_build_id() of a library built from them returns."""
    h = hashlib.sha256()
    for flag in extra_flags:
        h.update(flag.encode() + b"\0")
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".hpp", ".cpp", ".h")):
            h.update(name.encode() + b"\0")
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(f.read())
            h.update(b"\0")
    return h.hexdigest()[:16]


def _compile(src, out_dir=None, extra_flags=()):
    obj = os.path.join(out_dir or OUT_DIR, os.path.splitext(src)[0] + ".o")
    flags = list(extra_flags)
    if src == "api.hip":
        flags.append('-DMOE_BUILD_ID="%s"' % source_id(extra_flags))
    cmd = [hipcc()] + HIPCC_FLAGS + flags + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj, r.stderr


def build_library(verbose=False, out_dir=None, extra_flags=()):
    """out_dir / extra_flags: a second build beside the product's (tuning experiments with -D macros)."""
    out_dir = out_dir or OUT_DIR
    lib_path = os.path.join(out_dir, os.path.basename(LIB_PATH))
    os.makedirs(out_dir, exist_ok=True)
    # objects of sources that are no longer part of the library do not ship with it
    wanted = {os.path.splitext(src)[0] + ".o" for src in SOURCES}
    for name in os.listdir(out_dir):
        if name.endswith(".o") and name not in wanted:
            os.remove(os.path.join(out_dir, name))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(lambda src: _compile(src, out_dir, extra_flags), SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                print(err)
    # -Wl,--no-undefined: a launcher that a source file no longer defines fails the link here, not the first dlopen
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,--no-undefined", "-o", lib_path] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    return lib_path


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description="Builds libcandle_amd_moe.so; --out-dir / --flag: a second library beside the "
                                             "product's (measurement variants such as -DMOE_WHATIF=N of kernels_q4k_gemm.hip)")
    ap.add_argument("--out-dir", default=None)
    ap.add_argument("--flag", action="append", default=[])
    a = ap.parse_args()
    print(build_library(verbose=True, out_dir=a.out_dir, extra_flags=tuple(a.flag)))
