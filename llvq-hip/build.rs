// Links libllvq_hip.so (built by `make -C llvq_amd/csrc`, hipcc --offload-arch=gfx950).
// LLVQ_HIP_LIB_DIR names the directory that holds it; the library itself depends on
// libamdhip64 only, which the ROCm installation provides (ROCM_PATH, default /opt/rocm).
use std::env;

fn main() {
    println!("cargo:rerun-if-env-changed=LLVQ_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    if env::var_os("CARGO_FEATURE_LINK").is_none() {
        return;
    }
    let dir = env::var("LLVQ_HIP_LIB_DIR")
        .expect("set LLVQ_HIP_LIB_DIR to the directory that holds libllvq_hip.so");
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=llvq_hip");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    // the loader finds the library next to where it was built
    println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
}
