//! Links liblarql_hip.so (built by `python larql_amd/build.py`, which needs hipcc).
//! `LARQL_HIP_LIB_DIR` names the directory that holds it; the default is the sibling checkout's
//! `larql_amd/` directory.
use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=LARQL_HIP_LIB_DIR");
    let dir = env::var("LARQL_HIP_LIB_DIR").map(PathBuf::from).unwrap_or_else(|_| {
        PathBuf::from(env::var("CARGO_MANIFEST_DIR").expect("cargo sets CARGO_MANIFEST_DIR")).join("../larql_amd")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=larql_hip");
    // so that binaries find the library without LD_LIBRARY_PATH during development
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
}
