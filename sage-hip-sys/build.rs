// Tells cargo where libsage_hip.so lives and to link it dynamically.
//
// SAGE_HIP_LIB_DIR names the directory that holds libsage_hip.so (built by `python -m sage_amd.build`
// with hipcc for gfx950); by default the `sage_amd/` directory next to this crate.  The library itself
// links libamdhip64 and libhiprtc, which the loader finds through ROCm's own library path.
use std::env;
use std::path::PathBuf;

fn main() {
    let dir = env::var("SAGE_HIP_LIB_DIR").map(PathBuf::from).unwrap_or_else(|_| {
        PathBuf::from(env::var("CARGO_MANIFEST_DIR").unwrap()).join("..").join("sage_amd")
    });
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=sage_hip");
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
    println!("cargo:rerun-if-env-changed=SAGE_HIP_LIB_DIR");
    println!("cargo:rerun-if-changed=../include/sage_hip.h");
}
