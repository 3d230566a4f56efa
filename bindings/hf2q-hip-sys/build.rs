// Tells cargo where libhf2q_hip.so lives.  HF2Q_HIP_LIB_DIR names the directory that holds the library built by
// `python -m hf2q_amd.build` (it defaults to the in-tree location, ../../hf2q_amd relative to this crate).
use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=HF2Q_HIP_LIB_DIR");
    println!("cargo:rerun-if-changed=../../include/hf2q_hip.h");
    let dir = env::var("HF2Q_HIP_LIB_DIR").map(PathBuf::from).unwrap_or_else(|_| {
        PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("../../hf2q_amd")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=hf2q_hip");
    // the HIP runtime the library itself is linked against
    let rocm = env::var("ROCM_PATH").unwrap_or_else(|_| "/opt/rocm".to_string());
    println!("cargo:rustc-link-search=native={}/lib", rocm);
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
}
