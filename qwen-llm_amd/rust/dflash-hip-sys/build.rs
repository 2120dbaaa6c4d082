// Links the prebuilt library.  DFLASH_HIP_LIB_DIR names the directory that holds libdflash_hip.so
// (built by `python -c "import __graft_entry__ as g; g.build()"` into qwen-llm_amd/); ROCM_PATH the
// ROCm installation (default /opt/rocm) for the HIP runtime the library depends on.
use std::env;

fn main() {
    let lib_dir = env::var("DFLASH_HIP_LIB_DIR").expect("set DFLASH_HIP_LIB_DIR to the directory of libdflash_hip.so");
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={lib_dir}");
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=dflash_hip");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rerun-if-env-changed=DFLASH_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
}
