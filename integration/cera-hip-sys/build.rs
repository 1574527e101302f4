//! Link `libcera_hip.so`.
//!
//! `CERA_HIP_LIB_DIR` names the directory that holds it (the `cera_amd/lib/` folder of the
//! backend's own build, or wherever it was installed). The HIP runtime itself is a dependency of
//! that library, not of this crate, so nothing from ROCm is linked here.

use std::env;
use std::path::PathBuf;

fn main() {
    println!("cargo:rerun-if-env-changed=CERA_HIP_LIB_DIR");
    println!("cargo:rerun-if-changed=build.rs");

    let dir = match env::var_os("CERA_HIP_LIB_DIR") {
        Some(d) => PathBuf::from(d),
        None => panic!(
            "cera-hip-sys: set CERA_HIP_LIB_DIR to the directory that holds libcera_hip.so \
             (built by the hip backend's `__graft_entry__.build()` / `python -m cera_amd._build`)"
        ),
    };
    let lib = dir.join("libcera_hip.so");
    if !lib.exists() {
        panic!(
            "cera-hip-sys: {} does not exist (CERA_HIP_LIB_DIR={})",
            lib.display(),
            dir.display()
        );
    }
    println!("cargo:rustc-link-search=native={}", dir.display());
    println!("cargo:rustc-link-lib=dylib=cera_hip");
    // Let binaries find the library where it was linked from without LD_LIBRARY_PATH.
    println!("cargo:rustc-link-arg=-Wl,-rpath,{}", dir.display());
    // Dependents read this as DEP_CERA_HIP_LIB_DIR (e.g. to locate cera_hip_gfx950.hsaco).
    println!("cargo:lib_dir={}", dir.display());
}
