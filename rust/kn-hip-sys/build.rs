//! Links libknhip.so. No bindgen step (the declarations in src/lib.rs are written by hand against include/knhip.h),
//! no CUDA / HIP headers needed at build time: the library carries its own dependency on the ROCm runtime.
use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=KNHIP_LIB_DIR");
    let dir = env::var("KNHIP_LIB_DIR")
        .map(PathBuf::from)
        .expect("KNHIP_LIB_DIR must name the directory that holds libknhip.so (kyanite_amd/ after `python kyanite_amd/build.py`)");
    assert!(dir.join("libknhip.so").exists(), "no libknhip.so in {}", dir.display());
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=knhip");
    // so that binaries of dependent crates find the library without LD_LIBRARY_PATH
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
}
