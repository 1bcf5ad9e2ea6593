// Links libcandle_amd_moe.so (the HIP kernels behind include/candle_amd_moe.h).
//
// CANDLE_AMD_MOE_LIB_DIR names the directory that holds the built library (candle_amd/lib of the kernel
// repository after `python -m candle_amd.build`); without it the system's library path is searched.
use std::env;

fn main() {
    println!("cargo:rerun-if-env-changed=CANDLE_AMD_MOE_LIB_DIR");
    if let Ok(dir) = env::var("CANDLE_AMD_MOE_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        // so that test and example binaries find the library without LD_LIBRARY_PATH
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=candle_amd_moe");
}
