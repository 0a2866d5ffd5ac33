// Tells cargo where librllama_hip.so lives: RLLAMA_HIP_LIB_DIR, or ../../rllama_amd next to this crate (where
// `python -m rllama_amd.build` leaves it).
use std::env;
use std::path::PathBuf;

fn main() {
    let dir = env::var("RLLAMA_HIP_LIB_DIR").map(PathBuf::from).unwrap_or_else(|_| {
        PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("..").join("..").join("rllama_amd")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=rllama_hip");
    println!("cargo:rerun-if-env-changed=RLLAMA_HIP_LIB_DIR");
}
