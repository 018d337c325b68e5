// Points the linker at libfoundry_attn.so. FOUNDRY_ATTN_LIB_DIR names the directory that holds it (the in-tree build
// leaves it in test-burn_amd/); the HIP runtime it depends on comes from ROCM_PATH (default /opt/rocm).
use std::env;

fn main() {
    let dir = env::var("FOUNDRY_ATTN_LIB_DIR").unwrap_or_else(|_| "../../test-burn_amd".to_string());
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={}", dir);
    println!("cargo:rustc-link-search=native={}/lib", rocm);
    println!("cargo:rustc-link-lib=dylib=foundry_attn");
    println!("cargo:rerun-if-env-changed=FOUNDRY_ATTN_LIB_DIR");
    println!("cargo:rerun-if-changed=../../include/foundry_attn.h");
}
