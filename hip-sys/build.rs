// Links libmonarch_hip.so (built by `make -C monarch_amd/csrc`) and the HIP runtime.
// Mirrors the role of cuda-sys/build.rs in the reference: locate the native library,
// emit the link directives, export the library path to dependents.  No bindgen: the
// extern block in src/lib.rs is written by hand against include/monarch_hip.h and the
// test suite checks the two declaration sets against each other, name by name and type by type.
use std::env;
use std::path::PathBuf;

fn main() {
    let lib_dir = env::var("MONARCH_HIP_LIB_DIR").map(PathBuf::from).unwrap_or_else(|_| {
        PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("..").join("monarch_amd")
    });
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={}", lib_dir.display());
    println!("cargo:rustc-link-search=native={}/lib", rocm);
    println!("cargo:rustc-link-lib=dylib=monarch_hip");
    println!("cargo:rustc-link-lib=dylib=amdhip64");
    println!("cargo:LIB_PATH={}", lib_dir.display());  // DEP_MONARCH_HIP_LIB_PATH for dependents
    println!("cargo:rerun-if-env-changed=MONARCH_HIP_LIB_DIR");
    println!("cargo:rerun-if-env-changed=ROCM_PATH");
}
