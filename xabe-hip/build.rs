// Links libxabe_hip.so (built by `make -C llmxabe_amd/csrc`) and the HIP runtime.
// XABE_HIP_LIB_DIR: directory holding libxabe_hip.so (default: ../llmxabe_amd/lib); ROCM_PATH: default /opt/rocm.
fn main() {
    let lib_dir = std::env::var("XABE_HIP_LIB_DIR").unwrap_or_else(|_| {
        format!("{}/../llmxabe_amd/lib", std::env::var("CARGO_MANIFEST_DIR").unwrap())
    });
    let rocm = std::env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={lib_dir}");
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=xabe_hip");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:rerun-if-env-changed=XABE_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
}
