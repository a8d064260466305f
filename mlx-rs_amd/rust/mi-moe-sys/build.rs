// Link directives only: the library is built by its own Makefile with hipcc (there is no
// cmake step to drive, unlike mlx-sys/build.rs:6-45).
use std::env;

fn main() {
    // directory that holds libmi_moe.so
    let dir = env::var("MI_MOE_LIB_DIR").unwrap_or_else(|_| "/opt/mi_moe/lib".to_string());
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rerun-if-env-changed=MI_MOE_LIB_DIR");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
    println!("cargo:rustc-link-search=native={dir}");
    println!("cargo:rustc-link-search=native={rocm}/lib");
    println!("cargo:rustc-link-lib=dylib=mi_moe");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
}
